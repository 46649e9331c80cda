// Backward passes of the two memory-bound steps either side of the operator in the layer: the causal depthwise
// convolution (causal_conv1d_bwd, fla/modules/conv/triton/ops.py:147-249, kernels fla/modules/conv/triton/kernels.py:142-353
// and compute_dh0_kernel) and the normalisation with an output gate (layer_norm_gated_bwd,
// fla/modules/fused_norm_gate.py:541-650, kernels :192-453).  Both stream their operands once; the gradients of the
// parameters leave each workgroup as a row of partial sums in fp32 that the caller adds up (the reference does the same).
#include "gdn_common.h"
#include <type_traits>

namespace gdn {

// ---------------------------------------------------------------------------------------------
// convolution
//   z[t] = sum_j w[j] x[t - (W-1) + j] + b;  y[t] = act(z[t]) + residual[t];  final[i] = input at position len - W + i
//   dz[t] = dy[t] act'(z[t]);  dx[t] = sum_j w[j] dz[t + (W-1) - j]  (+ dht where t is one of the last W positions);
//   dw[j] = sum_t dz[t] x[t - (W-1) + j];  db = sum_t dz[t];  positions in front of the sequence belong to the initial state
// ---------------------------------------------------------------------------------------------
constexpr int CB_TOK = 4, CB_CX = 64, CB_TY = 4;       // a thread: 4 channels x 4 positions at a time; a wave: 256 channels; a workgroup: 4 waves
constexpr int CB_TILE = 64;                            // positions of a tile (the unit of the table for packed input)
constexpr int CB_VEC = 4;                              // Measured for bf16 at 32768 x 8192 (whole call): 4 channels x 4 positions (183 registers, two waves per
                                                       // SIMD) 331 us; 2 channels x 8 positions (150 registers, three waves) 338 us, with the next but one strip
                                                       // requested as well (168 registers) 380 us, with 16 / 4 tiles per workgroup instead of 8: 356 / 389 us.  Forms it replaced: a workgroup per tile of 64
                                                       // positions, every thread evaluating the W-1 dz behind its own positions again, 404 us; the same with those dz
                                                       // handed over through LDS (one barrier per tile) 420 - 450 us; tiles copied asynchronously into LDS two ahead
                                                       // (two barriers per tile) 472 us.  What counted was a loop without tested accesses: with them in the loop the
                                                       // compiler waits for the newest load before every use, and nothing is in flight while a wave computes.
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

// A number that is the same in every lane, moved to scalar registers: what is derived from it (the rows' base addresses,
// the step from row to row) is then scalar arithmetic, and a row is addressed as scalar base + one 32-bit lane offset.
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// What a thread needs of one tile: the inputs at its 8 positions and the W-1 in front of them (for z), and the output
// gradients at its positions.  The dz of the W-1 positions behind its own, which its last inputs feed as well, come from the
// thread that owns them (through LDS), not from a second evaluation of the activation.
template <typename T, int W>
struct ConvBwdRows {
    typedef T vec_t __attribute__((ext_vector_type(CB_VEC)));
    vec_t x[CB_TOK + W - 1];           // x[k]: position t0 - (W-1) + k
    vec_t dy[CB_TOK];                  // dy[i]: position t0 + i
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
    g.n = uniform_i64(g.n); g.it = uniform_i64(g.it); g.bos = uniform_i64(g.bos); g.len = uniform_i64(g.len);
    return g;
}

// The input at position s of the tile's sequence as the convolution sees it: the initial state in front of the sequence,
// zero behind it.
template <typename T>
__device__ __forceinline__ float conv_bwd_input(const ConvBwdParams& p, const ConvBwdTile& g, const T* xs, int c, int W, int64_t s) {
    if (s >= 0) return s < g.len ? (float)xs[s * p.stride_t] : 0.f;
    if (s < -(int64_t)(W - 1) || !p.initial_state) return 0.f;
    return load_scalar(p.initial_state, (g.n * p.D + c) * (int64_t)W + (W + s), p.state_dtype);
}

// Tiles that lie inside their sequence with W-1 positions in front are read without a test, so that all the loads of a
// thread are in flight together; the others (starts and ends of sequences) test every row, and read the initial state
// where a position lies in front of the sequence.
// With `held` (the strip behind this one in the same tile) the last W-1 rows of x are that strip's first W-1.
template <typename T, int W, bool HELD = false>
__device__ __forceinline__ void conv_bwd_fetch(const ConvBwdParams& p, const ConvBwdTile& g, int ty, int c0, ConvBwdRows<T, W>& r,
                                               const ConvBwdRows<T, W>& held) {
    constexpr int VEC = CB_VEC, NX = CB_TOK + W - 1, nx = HELD ? CB_TOK : NX;
    if constexpr (HELD) {
#pragma unroll
        for (int m = 0; m < W - 1; ++m) r.x[CB_TOK + m] = held.x[m];
    }
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    const int D = (int)p.D;
    if (g.it > 0 && (g.it + 1) * CB_TILE <= g.len) {
        // rows of the tile: a base that is the same for every lane (scalar registers, scalar arithmetic from row to row)
        // and one 32-bit offset per lane (the entry point bounds the strides accordingly)
        const char* xrow = (const char*)((const T*)p.x + (p.cu_seqlens ? g.bos * p.stride_t : g.n * p.stride_n)
                                         + (g.it * CB_TILE - (W - 1)) * p.stride_t);
        const char* dyrow = (const char*)((const T*)p.dy + (g.bos + g.it * CB_TILE) * D);
        const uint32_t xoff = (uint32_t)((ty * CB_TOK) * (int)p.stride_t + c0) * (uint32_t)sizeof(T);
        const uint32_t dyoff = (uint32_t)((ty * CB_TOK) * D + c0) * (uint32_t)sizeof(T);
#pragma unroll
        for (int k = 0; k < NX; ++k)
            if (k < nx) r.x[k] = *(const vec_t*)(xrow + (int64_t)k * p.stride_t * (int64_t)sizeof(T) + xoff);
#pragma unroll
        for (int i = 0; i < CB_TOK; ++i) r.dy[i] = *(const vec_t*)(dyrow + (int64_t)i * D * (int64_t)sizeof(T) + dyoff);
        return;
    }
    const int64_t t0 = g.it * CB_TILE + ty * CB_TOK;
    const T* xs = (const T*)p.x + (p.cu_seqlens ? g.bos * p.stride_t : g.n * p.stride_n) + c0;
    const T* dys = (const T*)p.dy + g.bos * D + c0;
#pragma unroll
    for (int k = 0; k < NX; ++k) {
        const int64_t s = t0 - (W - 1) + k;
        if (k >= nx) continue;
        r.x[k] = vec_t{};
        if (s >= 0 && s < g.len) r.x[k] = *(const vec_t*)(xs + s * p.stride_t);
        else if (s < 0 && p.initial_state) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) r.x[k][e] = (T)conv_bwd_input<T>(p, g, xs + e, c0 + e, W, s);
        }
    }
#pragma unroll
    for (int i = 0; i < CB_TOK; ++i) {
        r.dy[i] = vec_t{};
        if (t0 + i < g.len) r.dy[i] = *(const vec_t*)(dys + (t0 + i) * D);
    }
}

// dz[s] = dy[s] act'(z[s]) at the thread's 8 positions, with the sums for the parameters.
template <typename T, int W, bool ACT>
__device__ __forceinline__ void conv_bwd_dz(const ConvBwdRows<T, W>& r, const float (&wgt)[W][CB_VEC],
                                            const float (&bias)[CB_VEC], float (&dz)[CB_TOK + W - 1][CB_VEC],
                                            float (&dwacc)[W][CB_VEC], float (&dbacc)[CB_VEC]) {
#pragma unroll
    for (int i = 0; i < CB_TOK; ++i)
#pragma unroll
        for (int e = 0; e < CB_VEC; ++e) {
            float xf[W];
#pragma unroll
            for (int j = 0; j < W; ++j) xf[j] = (float)r.x[i + j][e];
            float d = (float)r.dy[i][e];                        // (zero past the end of the sequence)
            if constexpr (ACT) {
                float z = bias[e];
#pragma unroll
                for (int j = 0; j < W; ++j) z += wgt[j][e] * xf[j];
                d *= silu_grad(z);
            }
            dz[i][e] = d;
#pragma unroll
            for (int j = 0; j < W; ++j) dwacc[j][e] += d * xf[j];
            dbacc[e] += d;
        }
}

// dz at the W-1 positions from t1 on, evaluated from memory: only where no thread has just formed them (the strip a wave
// starts with).
template <typename T, int W>
__device__ __forceinline__ void conv_bwd_dz_behind(const ConvBwdParams& p, const ConvBwdTile& g, int64_t t1, int c0, const float (&wgt)[W][CB_VEC],
                                                   const float (&bias)[CB_VEC], float (&out)[W > 1 ? W - 1 : 1][CB_VEC]) {
    const int D = (int)p.D;
    const T* xs = (const T*)p.x + (p.cu_seqlens ? g.bos * p.stride_t : g.n * p.stride_n) + c0;
    const T* dys = (const T*)p.dy + g.bos * D + c0;
#pragma unroll
    for (int i = 0; i < W - 1; ++i)
#pragma unroll
        for (int e = 0; e < CB_VEC; ++e) {
            float d = 0.f;
            if (t1 + i < g.len) {
                d = (float)dys[(t1 + i) * D + e];
                if (p.act) {
                    float z = bias[e];
#pragma unroll
                    for (int j = 0; j < W; ++j) z += wgt[j][e] * conv_bwd_input<T>(p, g, xs + e, c0 + e, W, t1 + i - (W - 1) + j);
                    d *= silu_grad(z);
                }
            }
            out[i][e] = d;
        }
}

// dx[u] = sum_j w[j] dz[u + (W-1) - j] at the thread's 8 positions (+ dht where u is one of the sequence's last W).
template <typename T, int W>
__device__ __forceinline__ void conv_bwd_dx(const ConvBwdParams& p, const ConvBwdTile& g, int ty, int c0, const float (&wgt)[W][CB_VEC],
                                            const float (&dz)[CB_TOK + W - 1][CB_VEC]) {
    constexpr int VEC = CB_VEC;
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    const int D = (int)p.D;
    const int64_t t0 = g.it * CB_TILE + ty * CB_TOK, len = g.len;
    if ((g.it + 1) * CB_TILE <= len - (p.dht ? W : 0)) {   // a whole tile that the final state does not reach
        char* row = (char*)((T*)p.dx + (g.bos + g.it * CB_TILE) * D);
        const uint32_t off = (uint32_t)((ty * CB_TOK) * D + c0) * (uint32_t)sizeof(T);
#pragma unroll
        for (int i = 0; i < CB_TOK; ++i) {
            vec_t out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float a = 0.f;
#pragma unroll
                for (int j = 0; j < W; ++j) a += wgt[j][e] * dz[i + (W - 1) - j][e];
                out[e] = (T)a;
            }
            *(vec_t*)(row + (int64_t)i * D * (int64_t)sizeof(T) + off) = out;
        }
        return;
    }
    T* dxs = (T*)p.dx + g.bos * D + c0;
#pragma unroll
    for (int i = 0; i < CB_TOK; ++i) {
        const int64_t u = t0 + i;
        if (u >= len) continue;
        const bool in_final = p.dht && u >= len - W;            // this input is also entry u - (len - W) of the final state
        vec_t out;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float a = 0.f;
#pragma unroll
            for (int j = 0; j < W; ++j) a += wgt[j][e] * dz[i + (W - 1) - j][e];
            if (in_final) a += (float)((const T*)p.dht)[(g.n * D + c0 + e) * (int64_t)W + (u - (len - W))];
            out[e] = (T)a;
        }
        *(vec_t*)(dxs + u * D) = out;
    }
}

// A workgroup takes GDN_CONV_BWD_TILES_PER_PART consecutive tiles of its channels and keeps the sums for the parameters in
// registers across them: one row of partial sums per such run.  Each of its four waves owns a quarter of the run's
// positions and walks over it in strips of CB_TOK positions, LAST FIRST, with the rows of the next strip on their way into
// registers while it works on the current one; the waves never wait for each other and nothing passes through LDS.
// Walking backwards, a thread has just formed the W-1 dz behind its positions itself (only a wave's first strip evaluates
// them from memory), and inside a tile it already holds the W-1 rows of x in front of the strip it leaves.
template <typename T, int W>
__global__ __launch_bounds__(CB_CX * CB_TY, 2) void causal_conv1d_bwd_kernel(ConvBwdParams p) {
    constexpr int VEC = CB_VEC, H = W > 1 ? W - 1 : 1, STRIPS = CB_TILE / CB_TOK;      // strips of a tile
    static_assert(CB_CX == 64 && STRIPS % CB_TY == 0, "one wave per row of the block; the waves share a run evenly");
    __shared__ float red[W + 1][CB_TY][CB_CX * VEC];
    const int cx = threadIdx.x, wave = __builtin_amdgcn_readfirstlane((int)threadIdx.y);
    const int D = (int)p.D;
    const int64_t cblocks = (p.D + CB_CX * VEC - 1) / (CB_CX * VEC);
    const int64_t part = blockIdx.x / cblocks;
    const int c0 = (int)((blockIdx.x % cblocks) * CB_CX + cx) * VEC;
    const bool live = c0 < D;

    float dwacc[W][VEC], dbacc[VEC], wgt[W][VEC], bias[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        dbacc[e] = 0.f;
        bias[e] = live && p.bias ? load_scalar(p.bias, c0 + e, p.w_dtype) : 0.f;
#pragma unroll
        for (int j = 0; j < W; ++j) {
            dwacc[j][e] = 0.f;
            wgt[j][e] = live ? load_scalar(p.weight, (int64_t)(c0 + e) * W + j, p.w_dtype) : 0.f;
        }
    }
    const int64_t tile0 = part * GDN_CONV_BWD_TILES_PER_PART, tile_end = min(p.num_tiles, tile0 + GDN_CONV_BWD_TILES_PER_PART);
    const int per_wave = (int)(tile_end - tile0) * (STRIPS / CB_TY);     // strips per wave
    const int s_last = (wave + 1) * per_wave - 1;               // strip s of the run: tile tile0 + s / STRIPS, positions CB_TOK (s % STRIPS) ...
    const ConvBwdTile ga = conv_bwd_tile(p, tile0 + (s_last - (per_wave - 1)) / STRIPS), gb = conv_bwd_tile(p, tile0 + s_last / STRIPS);
    // The wave's strips lie in one sequence, the first of them W-1 positions or more from its start, the last one clear of
    // the positions that also feed the final state: nothing to test in the loop, whose waits for loads the compiler then
    // counts exactly (with the tested accesses of the other loop in it, it waits for the newest load before every use).
    const bool plain = ga.n == gb.n && gb.it - ga.it == (s_last / STRIPS) - ((s_last - (per_wave - 1)) / STRIPS) && ga.it > 0 &&
                       (gb.it + 1) * CB_TILE <= gb.len - (p.dht ? W : 0) && per_wave > 1;
    if (live && plain) {
        typedef T vec_t __attribute__((ext_vector_type(VEC)));
        int64_t pos = gb.it * CB_TILE + (s_last % STRIPS) * CB_TOK;      // first position of the strip in hand
        const int64_t xstep = p.stride_t * (int64_t)sizeof(T), dstep = (int64_t)D * (int64_t)sizeof(T);
        const uint32_t coff = (uint32_t)c0 * (uint32_t)sizeof(T);
        const char* xseq = (const char*)((const T*)p.x + (p.cu_seqlens ? gb.bos * p.stride_t : gb.n * p.stride_n));
        const char* dyseq = (const char*)((const T*)p.dy + gb.bos * D);
        char* dxseq = (char*)((T*)p.dx + gb.bos * D);
        vec_t xr[CB_TOK + W - 1], dyr[CB_TOK], xn[CB_TOK], dyn[CB_TOK];
#pragma unroll
        for (int k = 0; k < CB_TOK + W - 1; ++k) xr[k] = *(const vec_t*)(xseq + (pos - (W - 1) + k) * xstep + coff);
#pragma unroll
        for (int i = 0; i < CB_TOK; ++i) dyr[i] = *(const vec_t*)(dyseq + (pos + i) * dstep + coff);
        float first[H][VEC];                                    // the first W-1 dz of the strip behind the one in hand
        if constexpr (W > 1) {
            // from rows of their own: x up to position pos + CB_TOK - 1 is in hand, past the end of the sequence everything is zero
            vec_t xb[W - 1], dyb[W - 1];
#pragma unroll
            for (int i = 0; i < W - 1; ++i) {
                xb[i] = vec_t{}; dyb[i] = vec_t{};
                if (pos + CB_TOK + i < gb.len) {
                    xb[i] = *(const vec_t*)(xseq + (pos + CB_TOK + i) * xstep + coff);
                    dyb[i] = *(const vec_t*)(dyseq + (pos + CB_TOK + i) * dstep + coff);
                }
            }
#pragma unroll
            for (int i = 0; i < W - 1; ++i)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float d = (float)dyb[i][e];
                    if (p.act) {
                        float z = bias[e];
#pragma unroll
                        for (int j = 0; j < W; ++j) {           // input at position pos + CB_TOK + i - (W-1) + j
                            const int k = CB_TOK + i + j;       // as an index into xr (position pos - (W-1) + k)
                            z += wgt[j][e] * (k < CB_TOK + W - 1 ? (float)xr[k < CB_TOK + W - 1 ? k : 0][e] : (float)xb[k - (CB_TOK + W - 1) < W - 1 ? k - (CB_TOK + W - 1) : 0][e]);
                        }
                        d *= silu_grad(z);
                    }
                    first[i][e] = d;
                }
        }
        auto step = [&](auto ahead, auto act) {
            if constexpr (decltype(ahead)::value) {
#pragma unroll
                for (int k = 0; k < CB_TOK; ++k) xn[k] = *(const vec_t*)(xseq + (pos - CB_TOK - (W - 1) + k) * xstep + coff);
#pragma unroll
                for (int i = 0; i < CB_TOK; ++i) dyn[i] = *(const vec_t*)(dyseq + (pos - CB_TOK + i) * dstep + coff);
            }
            float dz[CB_TOK + W - 1][VEC];
#pragma unroll
            for (int i = 0; i < CB_TOK; ++i)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float xf[W];
#pragma unroll
                    for (int j = 0; j < W; ++j) xf[j] = (float)xr[i + j][e];
                    float d = (float)dyr[i][e];
                    if constexpr (decltype(act)::value) {
                        float z = bias[e];
#pragma unroll
                        for (int j = 0; j < W; ++j) z += wgt[j][e] * xf[j];
                        d *= silu_grad(z);
                    }
                    dz[i][e] = d;
#pragma unroll
                    for (int j = 0; j < W; ++j) dwacc[j][e] += d * xf[j];
                    dbacc[e] += d;
                }
#pragma unroll
            for (int i = 0; i < W - 1; ++i)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    dz[CB_TOK + i][e] = first[i][e];
                    first[i][e] = dz[i][e];
                }
#pragma unroll
            for (int i = 0; i < CB_TOK; ++i) {
                vec_t out;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float a = 0.f;
#pragma unroll
                    for (int j = 0; j < W; ++j) a += wgt[j][e] * dz[i + (W - 1) - j][e];
                    out[e] = (T)a;
                }
                *(vec_t*)(dxseq + (pos + i) * dstep + coff) = out;
            }
            if constexpr (decltype(ahead)::value) {
#pragma unroll
                for (int m = W - 2; m >= 0; --m) xr[CB_TOK + m] = xr[m];       // (last first: the two ranges overlap when W - 1 > CB_TOK)
#pragma unroll
                for (int k = 0; k < CB_TOK; ++k) { xr[k] = xn[k]; dyr[k] = dyn[k]; }
                pos -= CB_TOK;
            }
        };
        if (p.act) {
#pragma unroll 1
            for (int n = 0; n + 1 < per_wave; ++n) step(std::true_type{}, std::true_type{});
            step(std::false_type{}, std::true_type{});
        } else {
#pragma unroll 1
            for (int n = 0; n + 1 < per_wave; ++n) step(std::true_type{}, std::false_type{});
            step(std::false_type{}, std::false_type{});
        }
    } else if (live) {
        int s = s_last;
        ConvBwdRows<T, W> next;
        ConvBwdTile gnext = gb;
        conv_bwd_fetch<T, W>(p, gnext, s % STRIPS, c0, next, next);
        float first[H][VEC];                                    // the first W-1 dz of the strip taken before this one
#pragma unroll 1
        for (int n = 0; n < per_wave; ++n, --s) {
            const ConvBwdRows<T, W> cur = next;
            const ConvBwdTile g = gnext;
            const int ty = s % STRIPS;
            if (n + 1 < per_wave) {
                if (ty > 0) conv_bwd_fetch<T, W, true>(p, g, ty - 1, c0, next, cur);
                else {
                    gnext = conv_bwd_tile(p, tile0 + (s - 1) / STRIPS);
                    conv_bwd_fetch<T, W>(p, gnext, STRIPS - 1, c0, next, cur);
                }
            }
            float dz[CB_TOK + W - 1][VEC];
            if (p.act) conv_bwd_dz<T, W, true>(cur, wgt, bias, dz, dwacc, dbacc);
            else conv_bwd_dz<T, W, false>(cur, wgt, bias, dz, dwacc, dbacc);
            if constexpr (W > 1) {
                // the strip behind this one, if the sequence goes on there: what the last step left, or (first step) from memory
                const int64_t strip_end = g.it * CB_TILE + (ty + 1) * CB_TOK;
                if (strip_end >= g.len) {
#pragma unroll
                    for (int i = 0; i < W - 1; ++i)
#pragma unroll
                        for (int e = 0; e < VEC; ++e) first[i][e] = 0.f;
                } else if (n == 0) {
                    conv_bwd_dz_behind<T, W>(p, g, strip_end, c0, wgt, bias, first);
                }
#pragma unroll
                for (int i = 0; i < W - 1; ++i)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        dz[CB_TOK + i][e] = first[i][e];
                        first[i][e] = dz[i][e];
                    }
            }
            conv_bwd_dx<T, W>(p, g, ty, c0, wgt, dz);
        }
    }
    // sums over the workgroup's tokens (W taps and the bias), in a fixed order
#pragma unroll
    for (int q = 0; q <= W; ++q)
#pragma unroll
        for (int e = 0; e < VEC; ++e) red[q][threadIdx.y][cx * VEC + e] = q < W ? dwacc[q < W ? q : 0][e] : dbacc[e];
    __syncthreads();
    for (int q = threadIdx.y; q <= W; q += CB_TY) {
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
    GDN_CHECK_ARG(stride_x_t <= (1ll << 24), GDN_ERR_UNSUPPORTED, "%s: token stride %lld above 2^24 elements (a lane's offset inside a tile of 64 tokens is kept in 32 bits)",
                  who, (long long)stride_x_t);
    const uintptr_t pair = (uintptr_t)CB_VEC * (x_dtype == GDN_DTYPE_F32 ? 4 : 2);     // a thread reads its channels in one piece
    GDN_CHECK_ARG(D % CB_VEC == 0 && stride_x_t % CB_VEC == 0 && stride_x_n % CB_VEC == 0 && (uintptr_t)x % pair == 0 && (uintptr_t)dy % pair == 0 &&
                  (uintptr_t)dx % pair == 0, GDN_ERR_UNSUPPORTED, "%s: D and the strides of x must be multiples of %d and rows must start on %d-byte boundaries", who, CB_VEC, (int)pair);
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
