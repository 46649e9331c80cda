// Backward passes of the two memory-bound steps either side of the operator in the layer: the causal depthwise
// convolution (causal_conv1d_bwd, fla/modules/conv/triton/ops.py:147-249, kernels fla/modules/conv/triton/kernels.py:142-353
// and compute_dh0_kernel) and the normalisation with an output gate (layer_norm_gated_bwd,
// fla/modules/fused_norm_gate.py:541-650, kernels :192-453).  Both stream their operands once; the gradients of the
// parameters leave each workgroup as a row of partial sums in fp32 that the caller adds up (the reference does the same).
#include "gdn_common.h"

namespace gdn {

// ---------------------------------------------------------------------------------------------
// convolution
//   z[t] = sum_j w[j] x[t - (W-1) + j] + b;  y[t] = act(z[t]) + residual[t];  final[i] = input at position len - W + i
//   dz[t] = dy[t] act'(z[t]);  dx[t] = sum_j w[j] dz[t + (W-1) - j]  (+ dht where t is one of the last W positions);
//   dw[j] = sum_t dz[t] x[t - (W-1) + j];  db = sum_t dz[t];  positions in front of the sequence belong to the initial state
// ---------------------------------------------------------------------------------------------
constexpr int CB_TOK = 8, CB_CX = 32, CB_TY = 8;       // a thread: 2 channels x 8 positions; a workgroup: 32 channel pairs x 64 tokens
constexpr int CB_VEC = 2;                              // Two channels keep a thread at 134 registers (three waves per SIMD); measured for bf16 at
                                                       // 32768 x 3072: 4 channels (232 registers, two waves) 240 us, 2 channels 207 us; 8 channels or 16
                                                       // positions per thread: one wave per SIMD, 330 - 400 us; four waves by a register cap: spills, slower.
                                                       // (8 tiles per workgroup, GDN_CONV_BWD_TILES_PER_PART: 202 us against 207 us with 4.)
constexpr int CB_MAX_W = 8;

struct ConvBwdParams {
    const void* x; const void* weight; const void* bias; const void* initial_state; const void* dy; const void* dht;
    void* dx; float* dw_part; float* db_part; float* dh0;
    const void* cu_seqlens; const void* tile_table;
    int64_t B, T, D, N, NT, num_tiles;
    int64_t stride_n, stride_t;        // of x, in elements (channel stride 1)
    int W, w_dtype, state_dtype, act;
    bool cu32;
};

__device__ __forceinline__ float silu_grad(float z) {
    const float s = sigmoid_stream(z);
    return s * (1.f + z * (1.f - s));
}

// What a thread needs of one tile: the inputs at its 8 positions, the W-1 in front (for z) and the W-1 behind them (for
// the dz its last inputs feed), and the output gradients at its positions and the W-1 behind them.
template <typename T, int W>
struct ConvBwdRows {
    typedef T vec_t __attribute__((ext_vector_type(CB_VEC)));
    vec_t x[CB_TOK + 2 * (W - 1)];     // x[k]: position t0 - (W-1) + k
    vec_t dy[CB_TOK + W - 1];          // dy[i]: position t0 + i
};
struct ConvBwdTile { int64_t n, it, bos, len; };

__device__ __forceinline__ ConvBwdTile conv_bwd_tile(const ConvBwdParams& p, int64_t tile) {
    ConvBwdTile g;
    if (p.cu_seqlens) {
        g.n = load_index(p.tile_table, 2 * tile, p.cu32); g.it = load_index(p.tile_table, 2 * tile + 1, p.cu32);
        g.bos = load_index(p.cu_seqlens, g.n, p.cu32);
        g.len = load_index(p.cu_seqlens, g.n + 1, p.cu32) - g.bos;
    } else {
        g.n = tile / p.NT; g.it = tile % p.NT; g.bos = g.n * p.T; g.len = p.T;
    }
    return g;
}

// Tiles inside their sequence with W-1 positions in front and W behind them are read without a test, so that all the loads
// of a thread are in flight together; the others (starts and ends of sequences) test every row, and read the initial
// state where a position lies in front of the sequence.
template <typename T, int W>
__device__ __forceinline__ void conv_bwd_fetch(const ConvBwdParams& p, const ConvBwdTile& g, int ty, int c0, ConvBwdRows<T, W>& r) {
    constexpr int VEC = CB_VEC, NX = CB_TOK + 2 * (W - 1), NZ = CB_TOK + W - 1;
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    const int D = (int)p.D;
    const int64_t t0 = g.it * (CB_TOK * CB_TY) + ty * CB_TOK;
    const T* xs = (const T*)p.x + (p.cu_seqlens ? g.bos * p.stride_t : g.n * p.stride_n) + c0;
    const T* dys = (const T*)p.dy + g.bos * D + c0;
    if (g.it > 0 && (g.it + 1) * (CB_TOK * CB_TY) + W <= g.len) {
#pragma unroll
        for (int k = 0; k < NX; ++k) r.x[k] = *(const vec_t*)(xs + (t0 - (W - 1) + k) * p.stride_t);
#pragma unroll
        for (int i = 0; i < NZ; ++i) r.dy[i] = *(const vec_t*)(dys + (t0 + i) * D);
        return;
    }
#pragma unroll
    for (int k = 0; k < NX; ++k) {
        const int64_t s = t0 - (W - 1) + k;
        r.x[k] = vec_t{};
        if (s >= 0 && s < g.len) r.x[k] = *(const vec_t*)(xs + s * p.stride_t);
        else if (s < 0 && s >= -(W - 1) && p.initial_state) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) r.x[k][e] = (T)load_scalar(p.initial_state, (g.n * D + c0 + e) * (int64_t)W + (W + s), p.state_dtype);
        }
    }
#pragma unroll
    for (int i = 0; i < NZ; ++i) {
        r.dy[i] = vec_t{};
        if (t0 + i < g.len) r.dy[i] = *(const vec_t*)(dys + (t0 + i) * D);
    }
}

// The thread's 8 positions and the W-1 behind them in order, with the last W values of dz in registers (the loop is
// unrolled, so the window moves by renaming): dz[s] = dy[s] act'(z[s]);  dx[u] = sum_j w[j] dz[u + (W-1) - j].
template <typename T, int W>
__device__ __forceinline__ void conv_bwd_walk(const ConvBwdParams& p, const ConvBwdTile& g, int ty, int c0, const ConvBwdRows<T, W>& r,
                                              const float (&wgt)[W][CB_VEC], const float (&bias)[CB_VEC],
                                              float (&dwacc)[W][CB_VEC], float (&dbacc)[CB_VEC]) {
    constexpr int VEC = CB_VEC;
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    const int D = (int)p.D;
    const int64_t t0 = g.it * (CB_TOK * CB_TY) + ty * CB_TOK, len = g.len;
    T* dxs = (T*)p.dx + g.bos * D + c0;
    float dzw[W][VEC];                                          // dzw[j]: dz at position s - j
#pragma unroll
    for (int j = 0; j < W; ++j)
#pragma unroll
        for (int e = 0; e < VEC; ++e) dzw[j][e] = 0.f;
#pragma unroll
    for (int i = 0; i < CB_TOK + W - 1; ++i) {
        const int64_t s = t0 + i;
#pragma unroll
        for (int j = W - 1; j > 0; --j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) dzw[j][e] = dzw[j - 1][e];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float d = (float)r.dy[i][e];                        // (zero past the end of the sequence)
            if (p.act) {
                float z = bias[e];
#pragma unroll
                for (int j = 0; j < W; ++j) z += wgt[j][e] * (float)r.x[i + j][e];
                d *= silu_grad(z);
            }
            dzw[0][e] = d;
            if (i < CB_TOK) {                                   // (positions past this thread's own belong to the next thread's sums)
#pragma unroll
                for (int j = 0; j < W; ++j) dwacc[j][e] += d * (float)r.x[i + j][e];
                dbacc[e] += d;
            }
        }
        if (i >= W - 1) {
            const int64_t u = s - (W - 1);
            if (u < len) {
                const bool in_final = p.dht && u >= len - W;    // this input is also entry u - (len - W) of the final state
                vec_t out;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float a = 0.f;
#pragma unroll
                    for (int j = 0; j < W; ++j) a += wgt[j][e] * dzw[j][e];
                    if (in_final) a += (float)((const T*)p.dht)[(g.n * D + c0 + e) * (int64_t)W + (u - (len - W))];
                    out[e] = (T)a;
                }
                *(vec_t*)(dxs + u * D) = out;
            }
        }
    }
}

// A workgroup takes GDN_CONV_BWD_TILES_PER_PART consecutive tiles of its channels, one after the other, with the rows of the
// next tile on their way into registers while it works on the current one, and keeps the sums for the parameters in
// registers across them: one row of partial sums per such run.
template <typename T, int W>
__global__ __launch_bounds__(CB_CX * CB_TY, 2) void causal_conv1d_bwd_kernel(ConvBwdParams p) {
    constexpr int VEC = CB_VEC;
    __shared__ float red[W + 1][CB_TY][CB_CX * VEC];
    const int cx = threadIdx.x, ty = threadIdx.y;
    const int D = (int)p.D;
    const int64_t cblocks = (p.D + CB_CX * VEC - 1) / (CB_CX * VEC);
    const int64_t part = blockIdx.x / cblocks;
    const int c0 = (int)((blockIdx.x % cblocks) * CB_CX + cx) * VEC;

    float dwacc[W][VEC], dbacc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        dbacc[e] = 0.f;
#pragma unroll
        for (int j = 0; j < W; ++j) dwacc[j][e] = 0.f;
    }
    if (c0 < D) {
        float wgt[W][VEC], bias[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
#pragma unroll
            for (int j = 0; j < W; ++j) wgt[j][e] = load_scalar(p.weight, (int64_t)(c0 + e) * W + j, p.w_dtype);
            bias[e] = p.bias ? load_scalar(p.bias, c0 + e, p.w_dtype) : 0.f;
        }
        const int64_t tile0 = part * GDN_CONV_BWD_TILES_PER_PART, tile_end = min(p.num_tiles, tile0 + GDN_CONV_BWD_TILES_PER_PART);
        ConvBwdRows<T, W> next;
        ConvBwdTile gnext = conv_bwd_tile(p, tile0);
        conv_bwd_fetch<T, W>(p, gnext, ty, c0, next);
#pragma unroll 1
        for (int64_t tile = tile0; tile < tile_end; ++tile) {
            const ConvBwdRows<T, W> cur = next;
            const ConvBwdTile g = gnext;
            if (tile + 1 < tile_end) {
                gnext = conv_bwd_tile(p, tile + 1);
                conv_bwd_fetch<T, W>(p, gnext, ty, c0, next);
            }
            __builtin_amdgcn_sched_barrier(0);                  // (the loads are issued here, not where the scheduler finds room for them)
            conv_bwd_walk<T, W>(p, g, ty, c0, cur, wgt, bias, dwacc, dbacc);
        }
    }
    // sums over the workgroup's tokens (W taps and the bias), in a fixed order
#pragma unroll
    for (int q = 0; q <= W; ++q)
#pragma unroll
        for (int e = 0; e < VEC; ++e) red[q][ty][cx * VEC + e] = q < W ? dwacc[q < W ? q : 0][e] : dbacc[e];
    __syncthreads();
    for (int q = ty; q <= W; q += CB_TY) {
        if (c0 >= D || (q == W && !p.db_part)) continue;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float sum = 0.f;
#pragma unroll
            for (int r = 0; r < CB_TY; ++r) sum += red[q][r][cx * VEC + e];
            if (q < W) p.dw_part[(part * D + c0 + e) * W + q] = sum;
            else p.db_part[part * D + c0 + e] = sum;
        }
    }
}

// Gradient of the initial state [N, D, W] in fp32, one thread per (sequence, channel): entry i is the input at position
// i - W, read by the outputs at positions 0 .. i - 1; entries that a short sequence hands on to the final state take dht.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv1d_dh0_kernel(ConvBwdParams p) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.N * p.D) return;
    const int64_t n = i / p.D;
    const int d = (int)(i % p.D);
    const int W = p.W;
    int64_t bos, len;
    const T* xs;
    if (p.cu_seqlens) {
        bos = load_index(p.cu_seqlens, n, p.cu32);
        len = load_index(p.cu_seqlens, n + 1, p.cu32) - bos;
        xs = (const T*)p.x + bos * p.stride_t + d;
    } else {
        bos = n * p.T; len = p.T;
        xs = (const T*)p.x + n * p.stride_n + d;
    }
    float wgt[CB_MAX_W], dz[CB_MAX_W];
    for (int j = 0; j < W; ++j) wgt[j] = load_scalar(p.weight, (int64_t)d * W + j, p.w_dtype);
    const float bias = p.bias ? load_scalar(p.bias, d, p.w_dtype) : 0.f;
    auto input = [&](int64_t pos) -> float {
        if (pos >= 0) return pos < len ? (float)xs[pos * p.stride_t] : 0.f;
        return p.initial_state ? load_scalar(p.initial_state, i * W + (W + pos), p.state_dtype) : 0.f;
    };
    for (int s = 0; s < W - 1; ++s) {                           // dz at the first W-1 positions
        dz[s] = 0.f;
        if (s >= len) continue;
        float g = (float)((const T*)p.dy)[(bos + s) * p.D + d];
        if (p.act) {
            float z = bias;
            for (int j = 0; j < W; ++j) z += wgt[j] * input(s - (W - 1) + j);
            g *= silu_grad(z);
        }
        dz[s] = g;
    }
    for (int e = 0; e < W; ++e) {
        float a = 0.f;
        for (int j = 0; j < e; ++j) a += wgt[j] * dz[e - 1 - j];
        if (p.dht && e >= len && e - len < W) a += (float)((const T*)p.dht)[i * W + (e - len)];
        p.dh0[i * W + e] = a;
    }
}

template <typename T>
static int launch_conv_bwd(const ConvBwdParams& p, hipStream_t stream) {
    constexpr int VEC = CB_VEC;
    if (p.dx && p.num_tiles > 0) {
        const int64_t parts = (p.num_tiles + GDN_CONV_BWD_TILES_PER_PART - 1) / GDN_CONV_BWD_TILES_PER_PART;
        const int64_t blocks = ((p.D + CB_CX * VEC - 1) / (CB_CX * VEC)) * parts;
        if (blocks >= (1ll << 31)) {
            set_error("gdn_causal_conv1d_bwd: %lld workgroups exceed the grid limit", (long long)blocks);
            return GDN_ERR_UNSUPPORTED;
        }
        const dim3 grid((unsigned)blocks), block(CB_CX, CB_TY);
        switch (p.W) {
#define GDN_CONV_CASE(w) case w: hipLaunchKernelGGL((causal_conv1d_bwd_kernel<T, w>), grid, block, 0, stream, p); break;
            GDN_CONV_CASE(1) GDN_CONV_CASE(2) GDN_CONV_CASE(3) GDN_CONV_CASE(4)
            GDN_CONV_CASE(5) GDN_CONV_CASE(6) GDN_CONV_CASE(7) GDN_CONV_CASE(8)
#undef GDN_CONV_CASE
        }
        if (int rc = check_launch("causal_conv1d_bwd_kernel")) return rc;
    }
    if (p.dh0 && p.N * p.D > 0) {
        hipLaunchKernelGGL(causal_conv1d_dh0_kernel<T>, dim3((unsigned)((p.N * p.D + 255) / 256)), dim3(256), 0, stream, p);
        return check_launch("causal_conv1d_dh0_kernel");
    }
    return GDN_OK;
}

// ---------------------------------------------------------------------------------------------
// normalisation with an output gate
//   xhat = (r - mean) rstd;  yn = xhat w + b;  y = yn act(g)
//   dg = dy yn act'(g);  dyn = dy act(g);  dw = sum_rows dyn xhat;  db = sum_rows dyn;  wdy = dyn w
//   dr = (wdy - xhat mean_D(xhat wdy) - mean_D(wdy)) rstd  (+ the gradient of the residual stream); rms norm: no mean_D(wdy) term
// ---------------------------------------------------------------------------------------------
struct NormGateBwdParams {
    const void* dy; const void* x; const void* g; const void* weight; const void* bias;
    const float* mean; const float* rstd; const void* dresidual;
    void* dx; void* dg; float* dw_part; float* db_part;
    int64_t T, D, ld;                  // rows of D features, ld elements apart (a multiple of the 16-byte piece; dy is zero from D on)
    int w_dtype, act;
    bool rms;
};

template <int LANES>
__device__ __forceinline__ float lanes_sum(float v) {
#pragma unroll
    for (int m = LANES / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// A group of LANES lanes takes a row at a time (lane l: elements [(l + LANES i) VEC, +VEC), i < PIECES); the groups of all
// workgroups share the rows round robin and keep their parts of dw, db in registers until the end.
template <typename T, int LANES, int PIECES>
__global__ __launch_bounds__(256) void norm_gated_bwd_kernel(NormGateBwdParams p) {
    constexpr int VEC = 16 / sizeof(T), GROUPS = 256 / LANES;
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    __shared__ float red[GROUPS][LANES * PIECES * VEC];
    const int l = threadIdx.x % LANES, grp = threadIdx.x / LANES;
    const int D = (int)p.ld, Dtrue = (int)p.D;
    float wv[PIECES][VEC], bv[PIECES][VEC], dw[PIECES][VEC], db[PIECES][VEC];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int c = (l + LANES * i) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            wv[i][e] = (c + e < Dtrue && p.weight) ? load_scalar(p.weight, c + e, p.w_dtype) : 1.f;
            bv[i][e] = (c + e < Dtrue && p.bias) ? load_scalar(p.bias, c + e, p.w_dtype) : 0.f;
            dw[i][e] = 0.f; db[i][e] = 0.f;
        }
    }
    for (int64_t row = (int64_t)blockIdx.x * GROUPS + grp; row < p.T; row += (int64_t)gridDim.x * GROUPS) {
        const int64_t base = row * D;
        vec_t xv[PIECES], gv[PIECES], dyv[PIECES], drv[PIECES];
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int c = (l + LANES * i) * VEC;
            if (c < D) {
                xv[i] = *(const vec_t*)((const T*)p.x + base + c);
                gv[i] = *(const vec_t*)((const T*)p.g + base + c);
                dyv[i] = *(const vec_t*)((const T*)p.dy + base + c);
                if (p.dresidual) drv[i] = *(const vec_t*)((const T*)p.dresidual + base + c);
            }
        }
        const float mean = (p.rms || !p.mean) ? 0.f : p.mean[row], rstd = p.rstd[row];
        float xhat[PIECES][VEC], wdy[PIECES][VEC];
        float c1 = 0.f, c2 = 0.f;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int c = (l + LANES * i) * VEC;
            vec_t dgv;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                xhat[i][e] = 0.f; wdy[i][e] = 0.f;
                if (c < D) {
                    const float xh = ((float)xv[i][e] - mean) * rstd, yn = xh * wv[i][e] + bv[i][e];
                    const float gg = (float)gv[i][e], sg = sigmoid_f(gg), dyy = (float)dyv[i][e];
                    const float act = p.act == GDN_ACT_SILU ? gg * sg : sg;
                    const float dact = p.act == GDN_ACT_SILU ? sg * (1.f + gg * (1.f - sg)) : sg * (1.f - sg);
                    dgv[e] = (T)(dyy * yn * dact);
                    const float dyn = dyy * act;
                    dw[i][e] += dyn * xh;
                    db[i][e] += dyn;
                    xhat[i][e] = xh;
                    wdy[i][e] = dyn * wv[i][e];
                    c1 += xh * wdy[i][e];
                    c2 += wdy[i][e];
                }
            }
            if (c < D) *(vec_t*)((T*)p.dg + base + c) = dgv;
        }
        c1 = lanes_sum<LANES>(c1) / Dtrue;
        c2 = p.rms ? 0.f : lanes_sum<LANES>(c2) / Dtrue;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int c = (l + LANES * i) * VEC;
            if (c >= D) continue;
            vec_t out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float v = (wdy[i][e] - xhat[i][e] * c1 - c2) * rstd;
                if (p.dresidual) v += (float)drv[i][e];
                out[e] = (T)v;
            }
            *(vec_t*)((T*)p.dx + base + c) = out;
        }
    }
    // this workgroup's row of partial sums: the groups' parts added in a fixed order
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        float* dst = which ? p.db_part : p.dw_part;
        if (!dst) continue;                                     // (the same for the whole grid)
#pragma unroll
        for (int i = 0; i < PIECES; ++i)
#pragma unroll
            for (int e = 0; e < VEC; ++e) red[grp][(l + LANES * i) * VEC + e] = which ? db[i][e] : dw[i][e];
        __syncthreads();
        for (int c = threadIdx.x; c < D; c += 256) {
            float s = 0.f;
#pragma unroll
            for (int r = 0; r < GROUPS; ++r) s += red[r][c];
            dst[(int64_t)blockIdx.x * D + c] = s;
        }
        __syncthreads();
    }
}

template <typename T, int LANES, int PIECES>
static void launch_norm_bwd_rows(const NormGateBwdParams& p, int64_t parts, hipStream_t stream) {
    hipLaunchKernelGGL((norm_gated_bwd_kernel<T, LANES, PIECES>), dim3((unsigned)parts), dim3(256), 0, stream, p);
}

template <typename T>
static int launch_norm_bwd(const NormGateBwdParams& p, int64_t parts, hipStream_t stream) {
    constexpr int VEC = 16 / sizeof(T);
    const int64_t pieces = p.ld / VEC;
    if (pieces <= 8) launch_norm_bwd_rows<T, 8, 1>(p, parts, stream);
    else if (pieces <= 16) launch_norm_bwd_rows<T, 16, 1>(p, parts, stream);
    else if (pieces <= 32) launch_norm_bwd_rows<T, 32, 1>(p, parts, stream);
    else if (pieces <= 64) launch_norm_bwd_rows<T, 64, 1>(p, parts, stream);
    else if (pieces <= 128) launch_norm_bwd_rows<T, 64, 2>(p, parts, stream);
    else if (pieces <= 256) launch_norm_bwd_rows<T, 64, 4>(p, parts, stream);
    else launch_norm_bwd_rows<T, 64, (sizeof(T) == 4 ? 8 : 4)>(p, parts, stream);       // (fp32 rows only: checked by the entry point)
    return check_launch("norm_gated_bwd_kernel");
}

}  // namespace gdn

using namespace gdn;

static bool known_dtype(int d) { return d == GDN_DTYPE_BF16 || d == GDN_DTYPE_F16 || d == GDN_DTYPE_F32; }
static bool aligned16(const void* q) { return ((uintptr_t)q & 15) == 0; }

extern "C" int gdn_causal_conv1d_bwd(
    const void* x, const void* weight, const void* bias, const void* initial_state, const void* dy, const void* dht,
    void* dx, float* dw_part, float* db_part, float* dh0,
    const void* cu_seqlens, const void* tile_table,
    int64_t B, int64_t T, int64_t D, int64_t W, int64_t N, int64_t num_tiles, int64_t stride_x_n, int64_t stride_x_t,
    int x_dtype, int w_dtype, int state_dtype, int activation, uint32_t flags, void* stream) {
    const char* who = "gdn_causal_conv1d_bwd";
    GDN_CHECK_ARG(B >= 0 && T >= 0 && D >= 1 && N >= 0 && num_tiles >= 0, GDN_ERR_INVALID, "%s: bad sizes B=%lld T=%lld D=%lld N=%lld", who,
                  (long long)B, (long long)T, (long long)D, (long long)N);
    GDN_CHECK_ARG(W >= 1 && W <= CB_MAX_W, GDN_ERR_UNSUPPORTED, "%s: kernel size %lld outside 1..%d", who, (long long)W, CB_MAX_W);
    GDN_CHECK_ARG(known_dtype(x_dtype) && known_dtype(w_dtype) && known_dtype(state_dtype), GDN_ERR_UNSUPPORTED, "%s: unknown dtype", who);
    GDN_CHECK_ARG(activation == GDN_ACT_NONE || activation == GDN_ACT_SILU, GDN_ERR_UNSUPPORTED, "%s: activation must be none or silu", who);
    GDN_CHECK_ARG(!cu_seqlens || B == 1, GDN_ERR_INVALID, "%s: packed input needs B == 1", who);
    GDN_CHECK_ARG(cu_seqlens || N == B, GDN_ERR_INVALID, "%s: N must equal B for dense input", who);
    GDN_CHECK_ARG(!cu_seqlens || tile_table || num_tiles == 0, GDN_ERR_INVALID, "%s: packed input needs the table of 64-token tiles", who);
    GDN_CHECK_ARG(cu_seqlens || num_tiles == B * ((T + 63) / 64), GDN_ERR_INVALID, "%s: num_tiles does not match B and T", who);
    if (B * T == 0 && !dh0) return GDN_OK;
    GDN_CHECK_ARG(weight && (B * T == 0 || (x && dy && dx && dw_part)), GDN_ERR_INVALID, "%s: x, weight, dy, dx and dw_part are required", who);
    GDN_CHECK_ARG(!bias == !db_part, GDN_ERR_INVALID, "%s: db_part goes with bias", who);
    GDN_CHECK_ARG(!dh0 || initial_state, GDN_ERR_INVALID, "%s: dh0 needs initial_state", who);
    GDN_CHECK_ARG(D < (1ll << 31) && stride_x_t >= D, GDN_ERR_INVALID, "%s: token stride %lld below D", who, (long long)stride_x_t);
    const uintptr_t pair = (uintptr_t)CB_VEC * (x_dtype == GDN_DTYPE_F32 ? 4 : 2);     // a thread reads its two channels in one piece
    GDN_CHECK_ARG(D % CB_VEC == 0 && stride_x_t % CB_VEC == 0 && stride_x_n % CB_VEC == 0 && (uintptr_t)x % pair == 0 && (uintptr_t)dy % pair == 0 &&
                  (uintptr_t)dx % pair == 0, GDN_ERR_UNSUPPORTED, "%s: D and the strides of x must be even and rows must start on %d-byte boundaries", who, (int)pair);
    ConvBwdParams p{};
    p.x = x; p.weight = weight; p.bias = bias; p.initial_state = initial_state; p.dy = dy; p.dht = dht;
    p.dx = dx; p.dw_part = dw_part; p.db_part = db_part; p.dh0 = dh0;
    p.cu_seqlens = cu_seqlens; p.tile_table = tile_table;
    p.B = B; p.T = T; p.D = D; p.N = N; p.NT = (T + 63) / 64; p.num_tiles = num_tiles;
    p.stride_n = stride_x_n; p.stride_t = stride_x_t;
    p.W = (int)W; p.w_dtype = w_dtype; p.state_dtype = state_dtype; p.act = activation;
    p.cu32 = (flags & GDN_FLAG_CU_INT32) != 0;
    hipStream_t s = (hipStream_t)stream;
    if (x_dtype == GDN_DTYPE_BF16) return launch_conv_bwd<bf16_t>(p, s);
    if (x_dtype == GDN_DTYPE_F16) return launch_conv_bwd<f16_t>(p, s);
    return launch_conv_bwd<float>(p, s);
}

extern "C" int gdn_norm_gated_bwd(
    const void* dy, const void* x, const void* g, const void* weight, const void* bias,
    const float* mean, const float* rstd, const void* dresidual,
    void* dx, void* dg, float* dw_part, float* db_part,
    int64_t T, int64_t D, int64_t ld, int64_t parts,
    int x_dtype, int w_dtype, int activation, int is_rms_norm, void* stream) {
    const char* who = "gdn_norm_gated_bwd";
    GDN_CHECK_ARG(T >= 0 && D >= 1 && ld >= D && T < (1ll << 31), GDN_ERR_INVALID, "%s: bad sizes T=%lld D=%lld ld=%lld", who, (long long)T, (long long)D, (long long)ld);
    GDN_CHECK_ARG(parts >= 1 && parts <= 65535, GDN_ERR_INVALID, "%s: parts must be in 1..65535", who);
    GDN_CHECK_ARG(known_dtype(x_dtype) && known_dtype(w_dtype), GDN_ERR_UNSUPPORTED, "%s: unknown dtype", who);
    GDN_CHECK_ARG(activation == GDN_ACT_SILU || activation == GDN_ACT_SIGMOID, GDN_ERR_UNSUPPORTED, "%s: the gate must be swish/silu or sigmoid", who);
    const int64_t vec = x_dtype == GDN_DTYPE_F32 ? 4 : 8;
    GDN_CHECK_ARG(ld % vec == 0 && ld <= 2048, GDN_ERR_UNSUPPORTED, "%s: the row pitch must be a multiple of %lld up to 2048 (got %lld)", who,
                  (long long)vec, (long long)ld);
    GDN_CHECK_ARG(T == 0 || (dy && x && g && rstd && dx && dg), GDN_ERR_INVALID, "%s: dy, x, g, rstd, dx and dg are required", who);
    GDN_CHECK_ARG(T == 0 || is_rms_norm || mean, GDN_ERR_INVALID, "%s: layer norm needs the rows' means", who);
    GDN_CHECK_ARG(!weight == !dw_part && !bias == !db_part, GDN_ERR_INVALID, "%s: dw_part goes with weight and db_part with bias", who);
    GDN_CHECK_ARG(aligned16(dy) && aligned16(x) && aligned16(g) && aligned16(dx) && aligned16(dg) && aligned16(dresidual), GDN_ERR_UNSUPPORTED,
                  "%s: tensors must be 16-byte aligned", who);
    NormGateBwdParams p{dy, x, g, weight, bias, mean, rstd, dresidual, dx, dg, dw_part, db_part, T, D, ld, w_dtype, activation, is_rms_norm != 0};
    hipStream_t s = (hipStream_t)stream;
    if (x_dtype == GDN_DTYPE_BF16) return launch_norm_bwd<bf16_t>(p, parts, s);
    if (x_dtype == GDN_DTYPE_F16) return launch_norm_bwd<f16_t>(p, parts, s);
    return launch_norm_bwd<float>(p, parts, s);
}
