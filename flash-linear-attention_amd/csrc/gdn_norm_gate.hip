// Normalisation with an output gate over rows of D features: the step behind the gated delta rule in the
// layer (o_norm(o, g) per value head; fla/layers/gated_deltanet.py:355-359).
//
//   r = x (+ residual)                                 (r is also returned when asked for)
//   y = (r - mean) * rstd * weight + bias              (rms norm: mean = 0, rstd = 1/sqrt(mean(r^2) + eps))
//   y = y * g * sigmoid(g)   or   y * sigmoid(g)       (swish / sigmoid gate)
//
// Forward of layer_norm_gated_fwd (fla/modules/fused_norm_gate.py:456-538; kernels :36-108 and :125-189).
// Memory-bound: every element is read and written once.  Rows of up to 8 * 16 bytes per lane are held in
// registers by a group of 8..64 lanes (several rows per wave when D is small); longer or unaligned rows
// take a workgroup each and are read twice.
#include "gdn_common.h"

namespace gdn {

struct NormGateParams {
    const void* x; const void* g; const void* weight; const void* bias; const void* residual;
    void* y; void* residual_out; float* mean; float* rstd;
    int64_t T, D;
    float eps;
    int w_dtype, res_dtype, res_out_dtype, act;
    bool rms;
};

__device__ __forceinline__ void store_typed(void* p, int64_t i, int dtype, float v) {
    if (dtype == GDN_DTYPE_F32) ((float*)p)[i] = v;
    else if (dtype == GDN_DTYPE_BF16) ((bf16_t*)p)[i] = (bf16_t)v;
    else ((f16_t*)p)[i] = (f16_t)v;
}

__device__ __forceinline__ float gate_of(float y, float g, int act) {
    const float s = sigmoid_stream(g);
    return act == GDN_ACT_SILU ? y * g * s : y * s;
}

// Sum over the LANES lanes of a group (groups are aligned runs of lanes inside a wave).
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int m = LANES / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// Weights and biases of one 16-byte piece as fp32 (one vector load when they have the rows' element type).
template <typename T, int VEC>
__device__ __forceinline__ void load_params(const void* w, int c, int w_dtype, float fill, float (&out)[VEC]) {
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    constexpr int own = sizeof(T) == 4 ? GDN_DTYPE_F32 : (__is_same(T, bf16_t) ? GDN_DTYPE_BF16 : GDN_DTYPE_F16);
    if (!w) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) out[e] = fill;
    } else if (w_dtype == own && (((uintptr_t)w) & 15) == 0) {
        const vec_t v = *(const vec_t*)((const T*)w + c);
#pragma unroll
        for (int e = 0; e < VEC; ++e) out[e] = (float)v[e];
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) out[e] = load_scalar(w, c + e, w_dtype);
    }
}

// A group of LANES lanes holds ROWS rows at a time: lane l owns elements [(l + LANES * i) * VEC, +VEC) for
// i < PIECES of each.  All loads of the ROWS rows are issued before anything is reduced.
template <typename T, int LANES, int PIECES, int ROWS>
__global__ __launch_bounds__(256) void norm_gated_rows_kernel(NormGateParams p) {
    constexpr int VEC = 16 / sizeof(T);
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    const int l = threadIdx.x % LANES;
    // rows of a workgroup: round r covers 256 / LANES consecutive rows, one per group, so a wave's load is contiguous
    constexpr int GROUPS = 256 / LANES;
    const int64_t row0 = (int64_t)blockIdx.x * (GROUPS * ROWS) + threadIdx.x / LANES;
    const int D = (int)p.D;

    vec_t xv[ROWS][PIECES], gv[ROWS][PIECES];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int64_t base = min(row0 + r * GROUPS, p.T - 1) * D;     // rows past the end shadow the last row and store nothing
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int c = (l + LANES * i) * VEC;
            if (c < D) {
                xv[r][i] = *(const vec_t*)((const T*)p.x + base + c);
                gv[r][i] = *(const vec_t*)((const T*)p.g + base + c);
            }
        }
    }
    float v[ROWS][PIECES][VEC];
    float sum[ROWS], sq[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const bool live = row0 + r * GROUPS < p.T;
        const int64_t base = min(row0 + r * GROUPS, p.T - 1) * D;
        sum[r] = 0.f; sq[r] = 0.f;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int c = (l + LANES * i) * VEC;
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[r][i][e] = c < D ? (float)xv[r][i][e] : 0.f;
            if (c < D && p.residual) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) v[r][i][e] += load_scalar(p.residual, base + c + e, p.res_dtype);
            }
            if (c < D && p.residual_out && live) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) store_typed(p.residual_out, base + c + e, p.res_out_dtype, v[r][i][e]);
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) { sum[r] += v[r][i][e]; sq[r] += v[r][i][e] * v[r][i][e]; }
        }
    }
    float mean[ROWS], rstd[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        float var;
        if (p.rms) {
            mean[r] = 0.f;
            var = group_sum<LANES>(sq[r]) / D;
        } else {
            mean[r] = group_sum<LANES>(sum[r]) / D;
            float d2 = 0.f;
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                if ((l + LANES * i) * VEC < D) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) { const float d = v[r][i][e] - mean[r]; d2 += d * d; }
                }
            }
            var = group_sum<LANES>(d2) / D;
        }
        rstd[r] = 1.f / sqrtf(var + p.eps);
        if (l == 0 && row0 + r * GROUPS < p.T) {
            if (p.rstd) p.rstd[row0 + r * GROUPS] = rstd[r];
            if (p.mean && !p.rms) p.mean[row0 + r * GROUPS] = mean[r];
        }
    }
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int c = (l + LANES * i) * VEC;
        if (c >= D) continue;
        float wv[VEC], bv[VEC];
        load_params<T, VEC>(p.weight, c, p.w_dtype, 1.f, wv);
        load_params<T, VEC>(p.bias, c, p.w_dtype, 0.f, bv);
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            if (row0 + r * GROUPS >= p.T) continue;
            vec_t out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float y = (v[r][i][e] - mean[r]) * rstd[r] * wv[e] + bv[e];
                out[e] = (T)gate_of(y, (float)gv[r][i][e], p.act);
            }
            *(vec_t*)((T*)p.y + (row0 + r * GROUPS) * D + c) = out;
        }
    }
}

// Any D and alignment: one workgroup per row, element by element, the row read twice (three times for layer norm).
template <typename T>
__global__ __launch_bounds__(256) void norm_gated_long_kernel(NormGateParams p) {
    __shared__ float red[4];
    const int64_t base = (int64_t)blockIdx.x * p.D;
    const int D = (int)p.D;
    auto value = [&](int c) {
        float v = (float)((const T*)p.x)[base + c];
        if (p.residual) v += load_scalar(p.residual, base + c, p.res_dtype);
        return v;
    };
    auto block_sum = [&](float v) {
        v = group_sum<64>(v);
        __syncthreads();
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        return red[0] + red[1] + red[2] + red[3];
    };
    float sum = 0.f, sq = 0.f;
    for (int c = threadIdx.x; c < D; c += 256) {
        const float v = value(c);
        if (p.residual_out) store_typed(p.residual_out, base + c, p.res_out_dtype, v);
        sum += v; sq += v * v;
    }
    float mean = 0.f, var;
    if (p.rms) {
        var = block_sum(sq) / D;
    } else {
        mean = block_sum(sum) / D;
        float d2 = 0.f;
        for (int c = threadIdx.x; c < D; c += 256) { const float d = value(c) - mean; d2 += d * d; }
        var = block_sum(d2) / D;
    }
    const float rstd = 1.f / sqrtf(var + p.eps);
    if (threadIdx.x == 0) {
        if (p.rstd) p.rstd[blockIdx.x] = rstd;
        if (p.mean && !p.rms) p.mean[blockIdx.x] = mean;
    }
    for (int c = threadIdx.x; c < D; c += 256) {
        float y = (value(c) - mean) * rstd;
        if (p.weight) y *= load_scalar(p.weight, c, p.w_dtype);
        if (p.bias) y += load_scalar(p.bias, c, p.w_dtype);
        ((T*)p.y)[base + c] = (T)gate_of(y, (float)((const T*)p.g)[base + c], p.act);
    }
}

template <typename T, int LANES, int PIECES, int ROWS>
static void launch_rows(const NormGateParams& p, hipStream_t stream) {
    const int64_t rows_per_block = (256 / LANES) * ROWS;
    hipLaunchKernelGGL((norm_gated_rows_kernel<T, LANES, PIECES, ROWS>), dim3((unsigned)((p.T + rows_per_block - 1) / rows_per_block)),
                       dim3(256), 0, stream, p);
}

template <typename T>
static int launch_norm_gate(const NormGateParams& p, bool aligned, hipStream_t stream) {
    constexpr int VEC = 16 / sizeof(T);
    if (p.T == 0) return GDN_OK;
    const int64_t pieces = p.D / VEC;                         // 16-byte pieces per row (when D % VEC == 0)
    if (aligned && p.D % VEC == 0 && pieces <= 64 * 8) {
        if (pieces <= 8) launch_rows<T, 8, 1, 4>(p, stream);
        else if (pieces <= 16) launch_rows<T, 16, 1, 4>(p, stream);
        else if (pieces <= 32) launch_rows<T, 32, 1, 4>(p, stream);
        else if (pieces <= 64) launch_rows<T, 64, 1, 4>(p, stream);
        else if (pieces <= 128) launch_rows<T, 64, 2, 2>(p, stream);
        else if (pieces <= 256) launch_rows<T, 64, 4, 1>(p, stream);
        else launch_rows<T, 64, 8, 1>(p, stream);
    } else {
        hipLaunchKernelGGL(norm_gated_long_kernel<T>, dim3((unsigned)p.T), dim3(256), 0, stream, p);
    }
    return check_launch("norm_gated kernel");
}

}  // namespace gdn

using namespace gdn;

extern "C" int gdn_norm_gated_fwd(
    const void* x, const void* g, const void* weight, const void* bias, const void* residual,
    void* y, void* residual_out, float* mean, float* rstd,
    int64_t T, int64_t D, float eps,
    int x_dtype, int w_dtype, int res_dtype, int res_out_dtype, int activation, int is_rms_norm, void* stream) {
    auto is_dtype = [](int d) { return d == GDN_DTYPE_BF16 || d == GDN_DTYPE_F16 || d == GDN_DTYPE_F32; };
    GDN_CHECK_ARG((x && g && y) || T == 0, GDN_ERR_INVALID, "gdn_norm_gated_fwd: x, g and y are required");
    GDN_CHECK_ARG(T >= 0 && D >= 1 && T < (1ll << 31), GDN_ERR_INVALID, "gdn_norm_gated_fwd: bad sizes T=%lld D=%lld", (long long)T, (long long)D);
    GDN_CHECK_ARG(D <= 65536 / (x_dtype == GDN_DTYPE_F32 ? 4 : 2), GDN_ERR_UNSUPPORTED,
                  "gdn_norm_gated_fwd: rows of 64 KB and more are not supported (D=%lld)", (long long)D);
    GDN_CHECK_ARG(is_dtype(x_dtype) && is_dtype(w_dtype) && is_dtype(res_dtype) && is_dtype(res_out_dtype), GDN_ERR_UNSUPPORTED,
                  "gdn_norm_gated_fwd: unknown dtype");
    GDN_CHECK_ARG(activation == GDN_ACT_SILU || activation == GDN_ACT_SIGMOID, GDN_ERR_UNSUPPORTED,
                  "gdn_norm_gated_fwd: the gate must be swish/silu or sigmoid");
    NormGateParams p{x, g, weight, bias, residual, y, residual_out, mean, rstd, T, D, eps, w_dtype, res_dtype, res_out_dtype,
                     activation, is_rms_norm != 0};
    const bool aligned = (((uintptr_t)x | (uintptr_t)g | (uintptr_t)y) & 15) == 0;
    hipStream_t s = (hipStream_t)stream;
    if (x_dtype == GDN_DTYPE_BF16) return launch_norm_gate<bf16_t>(p, aligned, s);
    if (x_dtype == GDN_DTYPE_F16) return launch_norm_gate<f16_t>(p, aligned, s);
    return launch_norm_gate<float>(p, aligned, s);
}
