// Causal depthwise short convolution over [token][channel] rows: the step in front of the gated delta
// rule in the layer (q, k and v each pass through one; fla/layers/gated_deltanet.py:246-300).
//
//   y[t, d] = act( sum_{j < W} weight[d, j] * x[t - (W-1) + j, d] + bias[d] ) + residual[t, d]
//
// Positions before the start of a sequence read the sequence's initial state [N, D, W] (entry W + pos
// for pos = -1 .. -(W-1)) or zero.  Three kernels: prefill (causal_conv1d_fwd_kernel,
// fla/modules/conv/triton/kernels.py:37-139), the state left behind by a prefill
// (causal_conv1d_states_fwd_kernel, :520-582) and the one-token update of that state for decode
// (causal_conv1d_update_kernel, :356-421).  All three stream memory once.
#include "gdn_common.h"

namespace gdn {

constexpr int CONV_TOKENS = 8;         // tokens per thread (measured against 4 and 16: best)
constexpr int CONV_BX = 64, CONV_BY = 4;     // a workgroup: 64 channel groups x 4 token tiles (against 128 x 2, 256 x 1: best)
constexpr int CONV_MAX_W = 8;          // widest kernel

struct ConvParams {
    const void* x; const void* weight; const void* bias; const void* residual; const void* initial_state;
    void* y; void* final_state; const void* cu_seqlens;
    int64_t B, T, D, N, total;         // total = B*T tokens
    int64_t stride_n, stride_t;        // of x, in elements (channel stride is 1)
    int W, w_dtype, state_dtype, act;
    bool cu32;
};

// Sequence that holds global token `gt` (packed input): the last n with cu[n] <= gt.
__device__ __forceinline__ int64_t find_sequence(const void* cu, int64_t N, int64_t gt, bool cu32) {
    int64_t lo = 0, hi = N - 1;
    while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if (load_index(cu, mid, cu32) <= gt) lo = mid; else hi = mid - 1;
    }
    return lo;
}

template <typename T> struct dtype_of { static constexpr int value = GDN_DTYPE_F32; };
template <> struct dtype_of<bf16_t> { static constexpr int value = GDN_DTYPE_BF16; };
template <> struct dtype_of<f16_t> { static constexpr int value = GDN_DTYPE_F16; };

// A thread owns VEC adjacent channels (16 bytes when VECTOR, else one channel) and CONV_TOKENS consecutive
// tokens.  blockDim = (64 channel groups, 4 token tiles); the grid is flat: (groups / 64) x (tiles / 4) workgroups.
//
// Tiles that lie inside one sequence, W-1 tokens or more after its start, take the short way: the
// CONV_TOKENS + W-1 rows are requested at once (neighbouring tiles share W-1 of them through the caches)
// and contracted from registers.  Other tiles (sequence starts, ends of the input) go token by token and
// tap by tap, reading the initial state where a tap reaches in front of the sequence.
template <typename T, int W, bool VECTOR>
__global__ __launch_bounds__(256) void causal_conv1d_fwd_kernel(ConvParams p) {
    constexpr int VEC = VECTOR ? 16 / sizeof(T) : 1;
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    // workgroups are numbered channel block first, so those that run together cover whole rows of the same tokens
    const int64_t cblocks = (p.D + (int64_t)CONV_BX * VEC - 1) / ((int64_t)CONV_BX * VEC);
    const int c0 = (int)((blockIdx.x % cblocks) * CONV_BX + threadIdx.x) * VEC;
    int64_t gt0 = ((int64_t)(blockIdx.x / cblocks) * CONV_BY + threadIdx.y) * CONV_TOKENS;
    int64_t gt_end = min(gt0 + CONV_TOKENS, p.total);
    const int D = (int)p.D;
    const bool varlen = p.cu_seqlens != nullptr;
    if (varlen) {                                    // tokens outside [cu[0], cu[N]) belong to no sequence
        gt0 = max(gt0, load_index(p.cu_seqlens, 0, p.cu32));
        gt_end = min(gt_end, load_index(p.cu_seqlens, p.N, p.cu32));
    }
    if (c0 >= D || gt0 >= gt_end) return;

    // taps and bias of this thread's channels: weight rows are adjacent, VEC * W elements in one run
    float wgt[W][VEC], bias[VEC];
    if (VECTOR && p.w_dtype == dtype_of<T>::value && ((uintptr_t)p.weight & 15) == 0) {
        vec_t wraw[W];
#pragma unroll
        for (int j = 0; j < W; ++j) wraw[j] = *(const vec_t*)((const T*)p.weight + (int64_t)c0 * W + j * VEC);
#pragma unroll
        for (int i = 0; i < W * VEC; ++i) wgt[i % W][i / W] = (float)wraw[i / VEC][i % VEC];
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e)
#pragma unroll
            for (int j = 0; j < W; ++j) wgt[j][e] = load_scalar(p.weight, (int64_t)(c0 + e) * W + j, p.w_dtype);
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) bias[e] = p.bias ? load_scalar(p.bias, c0 + e, p.w_dtype) : 0.f;

    // the sequence of the first token and its bounds in global token numbers
    int64_t n, bos, eos;
    if (varlen) {
        n = find_sequence(p.cu_seqlens, p.N, gt0, p.cu32);
        bos = load_index(p.cu_seqlens, n, p.cu32);
        eos = load_index(p.cu_seqlens, n + 1, p.cu32);
    } else {
        n = gt0 / p.T; bos = n * p.T; eos = bos + p.T;
    }
    auto row_of = [&](int64_t gt) -> const T* {      // x row of global token gt of the current sequence
        return (const T*)p.x + (varlen ? gt * p.stride_t : n * p.stride_n + (gt - bos) * p.stride_t) + c0;
    };
    auto finish = [&](int64_t gt, float (&acc)[VEC], vec_t res) {
        vec_t out;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float a = acc[e] + bias[e];
            if (p.act) a = a * sigmoid_stream(a);
            if (p.residual) a += (float)res[e];
            out[e] = (T)a;
        }
        *(vec_t*)((T*)p.y + gt * D + c0) = out;
    };

    if (gt0 + CONV_TOKENS == gt_end && gt_end <= eos && gt0 - (W - 1) >= bos) {
        vec_t raw[CONV_TOKENS + W - 1];
        const T* first = row_of(gt0 - (W - 1));
#pragma unroll
        for (int i = 0; i < CONV_TOKENS + W - 1; ++i) raw[i] = *(const vec_t*)(first + i * p.stride_t);
#pragma unroll
        for (int u = 0; u < CONV_TOKENS; ++u) {
            float acc[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float a = 0.f;
#pragma unroll
                for (int j = 0; j < W; ++j) a += (float)raw[u + j][e] * wgt[j][e];
                acc[e] = a;
            }
            vec_t res = {};
            if (p.residual) res = *(const vec_t*)((const T*)p.residual + (gt0 + u) * D + c0);
            finish(gt0 + u, acc, res);
        }
        return;
    }

    for (int64_t gt = gt0; gt < gt_end; ++gt) {
        while (gt >= eos) {                          // first token of the next sequence (empty ones are skipped)
            ++n;
            bos = eos;
            eos = varlen ? load_index(p.cu_seqlens, n + 1, p.cu32) : bos + p.T;
        }
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
#pragma unroll
        for (int j = 0; j < W; ++j) {
            const int64_t src = gt - (W - 1) + j;
            if (src >= bos) {
                const vec_t v = *(const vec_t*)row_of(src);
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] += (float)v[e] * wgt[j][e];
            } else if (p.initial_state) {            // position src - bos = -1 .. -(W-1): state entry W + position
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    acc[e] += load_scalar(p.initial_state, (n * D + c0 + e) * (int64_t)W + (W + (src - bos)), p.state_dtype) * wgt[j][e];
            }
        }
        vec_t res = {};
        if (p.residual) res = *(const vec_t*)((const T*)p.residual + gt * D + c0);
        finish(gt, acc, res);
    }
}

// State after a prefill: the last W inputs of each sequence, older entries from the initial state or zero.
// One thread per (sequence, channel); W elements are contiguous in the state.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv1d_states_kernel(ConvParams p) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.N * p.D) return;
    const int64_t n = i / p.D;
    const int d = (int)(i % p.D);
    int64_t bos, len;
    const T* xs;
    if (p.cu_seqlens) {
        bos = load_index(p.cu_seqlens, n, p.cu32);
        len = load_index(p.cu_seqlens, n + 1, p.cu32) - bos;
        xs = (const T*)p.x + bos * p.stride_t + d;
    } else {
        len = p.T;
        xs = (const T*)p.x + n * p.stride_n + d;
    }
    T* out = (T*)p.final_state + i * p.W;
    for (int w = 0; w < p.W; ++w) {
        const int64_t pos = len - p.W + w;
        float v = 0.f;
        if (pos >= 0) v = (float)xs[pos * p.stride_t];
        else if (p.initial_state) v = load_scalar(p.initial_state, i * p.W + (w + len), p.state_dtype);
        out[w] = (T)v;
    }
}

struct ConvUpdateParams {
    const void* x; void* cache; const void* residual; const void* weight; const void* bias; void* y;
    int64_t N, D, stride_x_n, stride_y_n;
    int W, w_dtype, cache_dtype, act;
};

__device__ __forceinline__ void store_scalar(void* p, int64_t i, int dtype, float v) {
    if (dtype == GDN_DTYPE_F32) ((float*)p)[i] = v;
    else if (dtype == GDN_DTYPE_BF16) ((bf16_t*)p)[i] = (bf16_t)v;
    else ((f16_t*)p)[i] = (f16_t)v;
}

// One token per sequence: the cache [N, D, W] moves one place to the left, takes x at the end and is
// contracted with the weights.  One thread per (sequence, channel).  Without a cache the window is zero.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv1d_update_kernel(ConvUpdateParams p) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.N * p.D) return;
    const int64_t n = i / p.D;
    const int d = (int)(i % p.D);
    const float xv = (float)((const T*)p.x)[n * p.stride_x_n + d];
    float acc = 0.f;
    if (p.cache) {
        float win[CONV_MAX_W];
#pragma unroll
        for (int w = 0; w < CONV_MAX_W; ++w) {
            if (w >= p.W) break;
            win[w] = w + 1 < p.W ? load_scalar(p.cache, i * p.W + w + 1, p.cache_dtype) : xv;
        }
#pragma unroll
        for (int w = 0; w < CONV_MAX_W; ++w) {
            if (w >= p.W) break;
            acc += win[w] * (p.weight ? load_scalar(p.weight, (int64_t)d * p.W + w, p.w_dtype) : 1.f);
            store_scalar(p.cache, i * p.W + w, p.cache_dtype, win[w]);
        }
    }
    if (p.bias) acc += load_scalar(p.bias, d, p.w_dtype);
    if (p.act) acc = acc * sigmoid_stream(acc);
    if (p.residual) acc += (float)((const T*)p.residual)[n * p.D + d];
    ((T*)p.y)[n * p.stride_y_n + d] = (T)acc;
}

template <typename T, bool VECTOR>
static int launch_conv_fwd_w(const ConvParams& p, hipStream_t stream) {
    constexpr int VEC = VECTOR ? 16 / sizeof(T) : 1;
    const int64_t groups = (p.D + VEC - 1) / VEC, tiles = (p.total + CONV_TOKENS - 1) / CONV_TOKENS;
    const int64_t blocks = ((groups + CONV_BX - 1) / CONV_BX) * ((tiles + CONV_BY - 1) / CONV_BY);
    if (blocks >= (1ll << 31)) {
        set_error("gdn_causal_conv1d_fwd: %lld workgroups exceed the grid limit", (long long)blocks);
        return GDN_ERR_UNSUPPORTED;
    }
    const dim3 grid((unsigned)blocks), block(CONV_BX, CONV_BY);
    switch (p.W) {
#define GDN_CONV_CASE(w) case w: hipLaunchKernelGGL((causal_conv1d_fwd_kernel<T, w, VECTOR>), grid, block, 0, stream, p); break;
        GDN_CONV_CASE(1) GDN_CONV_CASE(2) GDN_CONV_CASE(3) GDN_CONV_CASE(4)
        GDN_CONV_CASE(5) GDN_CONV_CASE(6) GDN_CONV_CASE(7) GDN_CONV_CASE(8)
#undef GDN_CONV_CASE
    }
    return check_launch("causal_conv1d_fwd_kernel");
}

template <typename T>
static int launch_conv_fwd(const ConvParams& p, bool vec_ok, hipStream_t stream) {
    if (p.total > 0 && p.y) {
        if (int rc = vec_ok ? launch_conv_fwd_w<T, true>(p, stream) : launch_conv_fwd_w<T, false>(p, stream)) return rc;
    }
    if (p.final_state && p.N * p.D > 0) {
        hipLaunchKernelGGL(causal_conv1d_states_kernel<T>, dim3((unsigned)((p.N * p.D + 255) / 256)), dim3(256), 0, stream, p);
        return check_launch("causal_conv1d_states_kernel");
    }
    return GDN_OK;
}

}  // namespace gdn

using namespace gdn;

static bool is_dtype(int d) { return d == GDN_DTYPE_BF16 || d == GDN_DTYPE_F16 || d == GDN_DTYPE_F32; }

extern "C" int gdn_causal_conv1d_fwd(
    const void* x, const void* weight, const void* bias, const void* residual, const void* initial_state,
    void* y, void* final_state, const void* cu_seqlens,
    int64_t B, int64_t T, int64_t D, int64_t W, int64_t N, int64_t stride_x_n, int64_t stride_x_t,
    int x_dtype, int w_dtype, int state_dtype, int activation, uint32_t flags, void* stream) {
    GDN_CHECK_ARG((x && (y || final_state)) || B * T == 0, GDN_ERR_INVALID, "gdn_causal_conv1d_fwd: x and one of y, final_state are required");
    GDN_CHECK_ARG(!y || weight, GDN_ERR_INVALID, "gdn_causal_conv1d_fwd: y needs a weight");
    GDN_CHECK_ARG(B >= 0 && T >= 0 && D >= 1 && N >= 0, GDN_ERR_INVALID, "gdn_causal_conv1d_fwd: bad sizes B=%lld T=%lld D=%lld N=%lld",
                  (long long)B, (long long)T, (long long)D, (long long)N);
    GDN_CHECK_ARG(W >= 1 && W <= CONV_MAX_W, GDN_ERR_UNSUPPORTED, "gdn_causal_conv1d_fwd: kernel size %lld outside 1..%d", (long long)W, CONV_MAX_W);
    GDN_CHECK_ARG(is_dtype(x_dtype) && is_dtype(w_dtype) && is_dtype(state_dtype), GDN_ERR_UNSUPPORTED, "gdn_causal_conv1d_fwd: unknown dtype");
    GDN_CHECK_ARG(activation == GDN_ACT_NONE || activation == GDN_ACT_SILU, GDN_ERR_UNSUPPORTED, "gdn_causal_conv1d_fwd: activation must be none or silu");
    GDN_CHECK_ARG(!cu_seqlens || B == 1, GDN_ERR_INVALID, "gdn_causal_conv1d_fwd: packed input needs B == 1");
    GDN_CHECK_ARG(cu_seqlens || N == B, GDN_ERR_INVALID, "gdn_causal_conv1d_fwd: N must equal B for dense input");
    GDN_CHECK_ARG(D < (1ll << 31) && stride_x_t >= D, GDN_ERR_INVALID, "gdn_causal_conv1d_fwd: token stride %lld below D", (long long)stride_x_t);
    ConvParams p{};
    p.x = x; p.weight = weight; p.bias = bias; p.residual = residual; p.initial_state = initial_state;
    p.y = y; p.final_state = final_state; p.cu_seqlens = cu_seqlens;
    p.B = B; p.T = T; p.D = D; p.N = N; p.total = B * T;
    p.stride_n = stride_x_n; p.stride_t = stride_x_t;
    p.W = (int)W; p.w_dtype = w_dtype; p.state_dtype = state_dtype; p.act = activation;
    p.cu32 = (flags & GDN_FLAG_CU_INT32) != 0;
    const int64_t vec = x_dtype == GDN_DTYPE_F32 ? 4 : 8;
    auto aligned = [](const void* q) { return ((uintptr_t)q & 15) == 0; };
    // 16 bytes of channels per thread need every row to start on a 16-byte boundary
    const bool vec_ok = D % vec == 0 && stride_x_t % vec == 0 && stride_x_n % vec == 0 && aligned(x) && aligned(y) && aligned(residual);
    hipStream_t s = (hipStream_t)stream;
    if (x_dtype == GDN_DTYPE_BF16) return launch_conv_fwd<bf16_t>(p, vec_ok, s);
    if (x_dtype == GDN_DTYPE_F16) return launch_conv_fwd<f16_t>(p, vec_ok, s);
    return launch_conv_fwd<float>(p, vec_ok, s);
}

extern "C" int gdn_causal_conv1d_update(
    const void* x, void* cache, const void* residual, const void* weight, const void* bias, void* y,
    int64_t N, int64_t D, int64_t W, int64_t stride_x_n, int64_t stride_y_n,
    int x_dtype, int w_dtype, int cache_dtype, int activation, void* stream) {
    GDN_CHECK_ARG((x && y) || N == 0, GDN_ERR_INVALID, "gdn_causal_conv1d_update: x and y are required");
    GDN_CHECK_ARG(N >= 0 && D >= 1, GDN_ERR_INVALID, "gdn_causal_conv1d_update: bad sizes N=%lld D=%lld", (long long)N, (long long)D);
    GDN_CHECK_ARG(W >= 1 && W <= CONV_MAX_W, GDN_ERR_UNSUPPORTED, "gdn_causal_conv1d_update: kernel size %lld outside 1..%d", (long long)W, CONV_MAX_W);
    GDN_CHECK_ARG(is_dtype(x_dtype) && is_dtype(w_dtype) && is_dtype(cache_dtype), GDN_ERR_UNSUPPORTED, "gdn_causal_conv1d_update: unknown dtype");
    GDN_CHECK_ARG(activation == GDN_ACT_NONE || activation == GDN_ACT_SILU, GDN_ERR_UNSUPPORTED, "gdn_causal_conv1d_update: activation must be none or silu");
    if (N * D == 0) return GDN_OK;
    ConvUpdateParams p{x, cache, residual, weight, bias, y, N, D, stride_x_n, stride_y_n, (int)W, w_dtype, cache_dtype, activation};
    const dim3 grid((unsigned)((N * D + 255) / 256)), block(256);
    hipStream_t s = (hipStream_t)stream;
    if (x_dtype == GDN_DTYPE_BF16) hipLaunchKernelGGL(causal_conv1d_update_kernel<bf16_t>, grid, block, 0, s, p);
    else if (x_dtype == GDN_DTYPE_F16) hipLaunchKernelGGL(causal_conv1d_update_kernel<f16_t>, grid, block, 0, s, p);
    else hipLaunchKernelGGL(causal_conv1d_update_kernel<float>, grid, block, 0, s, p);
    return check_launch("causal_conv1d_update_kernel");
}
