// Chunked prefill of the gated delta rule for gfx950 (MI355X): 64-token chunks, K = V = 128.
//
// Two kernels, both built on v_mfma_f32_16x16x32 (bf16 or f16 operands, fp32 accumulate):
//
//  gdn_chunk_prepare_kernel   one workgroup per (chunk, v-head); everything that does not
//      depend on the running state:  G = cumsum(g)/ln2,  L = beta*(K K^T)*2^(G_i-G_j) (i>j),
//      A = (I+L)^-1 in fp32 (16x16 forward substitution on the diagonal blocks, fp32-MFMA block
//      merges),  w = A (beta*2^G*k),  u = A (beta*v),  P = tril(q k^T * 2^(G_i-G_j)).
//      Results are written in the exact register order ("fragments") in which the second
//      kernel feeds them to the matrix cores, so that kernel needs no transposes.
//
//  gdn_chunk_scan_kernel      one workgroup per (sequence, v-head, slab of value columns);
//      walks the chunks in order with the fp32 state S[K, slab] in registers:
//      v_new = u - w S;  o = scale*((q S)*2^G + P v_new);  S = 2^G_last S + k^T (v_new*2^(G_last-G)).
//      Per-chunk states and v_new never go to memory.
//
// MFMA register layout used throughout (wave64, lane l, c16 = l%16, g = l/16):
//   A operand (M x 32): lane holds row c16, 8 contraction indices chosen by g;
//   B operand (32 x N): lane holds column c16, the same 8 contraction indices;
//   C/D (16 x 16):      lane holds column c16, rows 4g..4g+3.
// Any assignment of contraction indices to (g, element) is valid as long as A and B agree.
// The scan kernel uses {16a+4g+r} U {16b+4g+r} for a pair of 16-row tiles (a, b): that is
// exactly how a C/D result is spread over lanes, so an accumulator can be converted in
// place into the B operand of the next product.
#include "gdn_common.h"

namespace gdn {

constexpr int CH = 64;                       // chunk length
constexpr float RCP_LN2_F = 1.4426950216f;   // fla/ops/utils/constant.py:10

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    typedef bf16x8 V8;
    typedef bf16x4 V4;
    static __device__ __forceinline__ f32x4 run(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<f16_t> {
    typedef f16x8 V8;
    typedef f16x4 V4;
    static __device__ __forceinline__ f32x4 run(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

// Per-chunk workspace written by the prepare kernel (element counts for K = V = 128):
//   G   fp32 [NC][HV][64]                   chunk-local gate cumsum in log2 units
//   Wf  T    [NC][HV][4 tt][4 s][64][8]     w rows of t-tile tt, key tiles (2s, 2s+1)
//   Uf  T    [NC][HV][8 n ][4 tt][64][4]    u, C/D layout of tile (t-tile tt, value tile n)
//   KTf T    [NC][H ][8 m ][2 s][64][8]     k^T rows of key tile m, t-tiles (2s, 2s+1)
//   Pf  T    [NC][HV][4 tt][2 s][64][8]     P rows of t-tile tt, t-tiles (2s, 2s+1) as columns
struct ChunkWs {
    float* G;
    void* Wf;
    void* Uf;
    void* KTf;
    void* Pf;
};
constexpr int64_t WS_W = 8192, WS_U = 8192, WS_KT = 8192, WS_P = 4096;   // elements per (chunk, head)

static size_t ws_align(size_t x) { return (x + 255) & ~(size_t)255; }

static size_t ws_layout(int64_t NC, int64_t H, int64_t HV, char* base, ChunkWs* ws) {
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += ws_align(bytes); return base ? (void*)(base + o) : nullptr; };
    void* G = take((size_t)NC * HV * CH * 4);
    void* Wf = take((size_t)NC * HV * WS_W * 2);
    void* Uf = take((size_t)NC * HV * WS_U * 2);
    void* KTf = take((size_t)NC * H * WS_KT * 2);
    void* Pf = take((size_t)NC * HV * WS_P * 2);
    if (ws) { ws->G = (float*)G; ws->Wf = Wf; ws->Uf = Uf; ws->KTf = KTf; ws->Pf = Pf; }
    return off;
}

struct ChunkParams {
    const void* q; const void* k; const void* v; const void* g; const void* beta;
    const float* h0; float* ht; void* o;
    const void* cu_seqlens; const void* chunk_table; const void* chunk_offsets;
    ChunkWs ws;
    int64_t T; int H, HV; int64_t N; int64_t NT;       // NT: chunks per sequence (dense input)
    float scale; int gb_dtype; uint32_t flags;
    int nslab; int64_t NH;
};

// Workgroup barrier that only waits for this wave's LDS traffic.  __syncthreads() also drains
// the vector-memory counter, which would serialise the global prefetch of the next chunk
// behind every barrier of the current one.
#ifndef GDN_EXP
#define GDN_EXP 0
#endif
__device__ __forceinline__ void lds_barrier() {
    if (GDN_EXP == 3) return;
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 16x16 product of fp32 matrices held in LDS on the fp32 matrix cores:
// C = A[16 x 4*nk] * B[4*nk x 16]; result in C/D layout.
__device__ __forceinline__ f32x4 mm16_f32(const float* A, int lda, const float* B, int ldb, int nk, int c16, int g) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int kk = 0; kk < nk; ++kk) {
        const float a = A[c16 * lda + 4 * kk + g];
        const float b = B[(4 * kk + g) * ldb + c16];
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc, 0, 0, 0);
    }
    return acc;
}

// ============================================================================================
// prepare kernel
// ============================================================================================
constexpr int NP = 128 + 8;     // pitch (elements) of the staged 64x128 tiles: 272 B rows, conflict-free 16 B reads
constexpr int LP = 68;          // pitch (floats) of the 64x64 fp32 matrices
constexpr size_t PREP_SMEM = 3 * CH * NP * 2 + CH * LP * 4 + 3 * CH * 4;

template <typename T>
__global__ __launch_bounds__(256) void gdn_chunk_prepare_kernel(ChunkParams p) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    T* k_nat = (T*)smem;                        // [64][NP] keys, token-major
    T* q_nat = k_nat + CH * NP;                 // [64][NP] queries; the region is reused for X below
    T* v_nat = q_nat + CH * NP;                 // [64][NP] values
    float* sL = (float*)(v_nat + CH * NP);      // [64][LP] L (strictly lower)
    float* sX = (float*)q_nat;                  // [64][LP] (I+L)^-1, same bytes as q_nat (64*136*2 == 64*68*4)
    float* sG = sL + CH * LP;                   // [64] cumulative gate (log2)
    float* sB = sG + CH;                        // [64] beta
    float* sBG = sB + CH;                       // [64] beta * 2^G

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    const int64_t ci = blockIdx.x;
    const int hv = blockIdx.y;
    const int H = p.H, HV = p.HV;
    const int h = hv / (HV / H);
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;

    int64_t tok0;
    int valid;
    if (p.cu_seqlens) {
        const int64_t n = load_index(p.chunk_table, 2 * ci, cu32), it = load_index(p.chunk_table, 2 * ci + 1, cu32);
        const int64_t bos = load_index(p.cu_seqlens, n, cu32), eos = load_index(p.cu_seqlens, n + 1, cu32);
        tok0 = bos + it * CH;
        valid = (int)min((int64_t)CH, eos - tok0);
    } else {
        const int64_t b = ci / p.NT, it = ci % p.NT;
        tok0 = b * p.T + it * CH;
        valid = (int)min((int64_t)CH, p.T - it * CH);
    }

    // ---- stage k, q, v (rows past the end of the sequence are zero) ----
    const T* kg = (const T*)p.k + (tok0 * H + h) * 128;
    const T* qg = (const T*)p.q + (tok0 * H + h) * 128;
    const T* vg = (const T*)p.v + (tok0 * HV + hv) * 128;
    u32x4 rk[4], rq[4], rv[4];
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int row = ps * 16 + (tid >> 4), col = (tid & 15) * 8;
        const u32x4 z = {0u, 0u, 0u, 0u};
        rk[ps] = rq[ps] = rv[ps] = z;
        if (row < valid) {
            rk[ps] = *(const u32x4*)(kg + (int64_t)row * H * 128 + col);
            rq[ps] = *(const u32x4*)(qg + (int64_t)row * H * 128 + col);
            rv[ps] = *(const u32x4*)(vg + (int64_t)row * HV * 128 + col);
        }
    }
    // ---- gates: inclusive scan over the chunk (wave 0, one token per lane) ----
    if (w == 0) {
        float x = 0.f, b = 0.f;
        if (lane < valid) {
            x = load_scalar(p.g, (tok0 + lane) * HV + hv, p.gb_dtype);
            b = load_scalar(p.beta, (tok0 + lane) * HV + hv, p.gb_dtype);
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float y = __shfl_up(x, off, 64);
            if (lane >= off) x += y;
        }
        x *= RCP_LN2_F;
        sG[lane] = x;
        sB[lane] = b;
        sBG[lane] = b * exp2f(x);
        p.ws.G[(ci * HV + hv) * CH + lane] = x;
    }
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int row = ps * 16 + (tid >> 4), col = (tid & 15) * 8;
        *(u32x4*)(k_nat + row * NP + col) = rk[ps];
        *(u32x4*)(q_nat + row * NP + col) = rq[ps];
        *(u32x4*)(v_nat + row * NP + col) = rv[ps];
    }
    __syncthreads();

    // ---- L tiles of row-tile w (K K^T, gated, beta-scaled, strictly lower) ----
    {
        V8 ka[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) ka[s] = *(const V8*)(k_nat + (16 * w + c16) * NP + 32 * s + 8 * g);
        for (int tj = 0; tj < 4; ++tj) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            if (tj <= w) {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const V8 kb = *(const V8*)(k_nat + (16 * tj + c16) * NP + 32 * s + 8 * g);
                    acc = Mma<T>::run(ka[s], kb, acc);
                }
            }
            const int j = 16 * tj + c16;
            const float gj = sG[j];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 16 * w + 4 * g + r;
                // select, never multiply by a mask: 2^(G_i-G_j) may overflow above the diagonal
                const float val = (i > j) ? sB[i] * acc[r] * exp2f(sG[i] - gj) : 0.f;
                sL[i * LP + j] = val;
            }
        }
    }
    // ---- P^T tiles of column-tile tt = 3-w (k_j . q_t, gated, lower incl. diagonal), straight to memory ----
    {
        const int tt = 3 - w;
        V8 qb[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) qb[s] = *(const V8*)(q_nat + (16 * tt + c16) * NP + 32 * s + 8 * g);
        const int t = 16 * tt + c16;
        const float gt = sG[t];
        T* pf = (T*)p.ws.Pf + (ci * HV + hv) * WS_P;
        for (int sp = 0; sp <= tt / 2; ++sp) {
            V8 frag;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int tj = 2 * sp + half;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                if (tj <= tt) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const V8 ka = *(const V8*)(k_nat + (16 * tj + c16) * NP + 32 * s + 8 * g);
                        acc = Mma<T>::run(ka, qb[s], acc);
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = 16 * tj + 4 * g + r;
                    const float val = (t >= j) ? acc[r] * exp2f(gt - sG[j]) : 0.f;
                    frag[half * 4 + r] = from_f32<T>(val);
                }
            }
            *(V8*)(pf + ((tt * 2 + sp) * 64 + lane) * 8) = frag;
        }
    }
    __syncthreads();     // L complete; q_nat is dead from here on and becomes X

    // ---- X = (I+L)^-1: 16x16 diagonal blocks by forward substitution (column c16 per lane) ----
    {
        const int b0 = 16 * w;
        float x[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float acc = (i == c16) ? 1.f : 0.f;
#pragma unroll
            for (int j = 0; j < i; ++j) acc -= sL[(b0 + i) * LP + b0 + j] * x[j];
            x[i] = acc;
        }
        if (g == 0) {
#pragma unroll
            for (int i = 0; i < 16; ++i) sX[(b0 + i) * LP + b0 + c16] = x[i];
        }
        // zero tile above the diagonal inside each 32x32 diagonal block
        if ((w & 1) == 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) sX[(b0 + 4 * g + r) * LP + b0 + 16 + c16] = 0.f;
        }
    }
    __syncthreads();
    // ---- merge 16 -> 32: X[hi][lo] = -X[hi][hi] (L[hi][lo] X[lo][lo]); pairs (1,0) and (3,2) ----
    // (waves 2,3 repeat the work of waves 0,1 so that the barriers stay block-uniform)
    {
        const int pr = w & 1, hi = 2 * pr + 1, lo = 2 * pr;
        float* tmp = sX + 32 + 16 * pr;                     // rows 0..15 of the unused upper-right block
        f32x4 y = mm16_f32(sL + (16 * hi) * LP + 16 * lo, LP, sX + (16 * lo) * LP + 16 * lo, LP, 4, c16, g);
        if (w < 2) {
#pragma unroll
            for (int r = 0; r < 4; ++r) tmp[(4 * g + r) * LP + c16] = y[r];
        }
        __syncthreads();
        f32x4 z = mm16_f32(sX + (16 * hi) * LP + 16 * hi, LP, tmp, LP, 4, c16, g);
        if (w < 2) {
#pragma unroll
            for (int r = 0; r < 4; ++r) sX[(16 * hi + 4 * g + r) * LP + 16 * lo + c16] = -z[r];
        }
    }
    __syncthreads();
    // ---- merge 32 -> 64: X[32:64][0:32] = -X[32:64][32:64] (L[32:64][0:32] X[0:32][0:32]) ----
    {
        const int a = w >> 1, b = w & 1;
        float* tmp2 = sX + 32;                              // rows 0..31, columns 32..63
        f32x4 y = mm16_f32(sL + (32 + 16 * a) * LP, LP, sX + 16 * b, LP, 8, c16, g);
        __syncthreads();                                    // level-1 temporaries (same region) fully consumed
#pragma unroll
        for (int r = 0; r < 4; ++r) tmp2[(16 * a + 4 * g + r) * LP + 16 * b + c16] = y[r];
        __syncthreads();
        f32x4 z = mm16_f32(sX + (32 + 16 * a) * LP + 32, LP, tmp2 + 16 * b, LP, 8, c16, g);
#pragma unroll
        for (int r = 0; r < 4; ++r) sX[(32 + 16 * a + 4 * g + r) * LP + 16 * b + c16] = -z[r];
    }
    __syncthreads();

    // ---- w^T = k^T (diag(beta 2^G) X^T) and u = (X diag(beta)) v for t-tile w ----
    const int ns = (w >= 2) ? 2 : 1;         // X is lower triangular: columns >= 32 matter only for rows >= 32
    V8 fw[2], fu[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        if (s < ns) {
            const float* xr = sX + (16 * w + c16) * LP + 32 * s + 8 * g;
            const f32x4 x0 = *(const f32x4*)xr, x1 = *(const f32x4*)(xr + 4);
            const f32x4 bg0 = *(const f32x4*)(sBG + 32 * s + 8 * g), bg1 = *(const f32x4*)(sBG + 32 * s + 8 * g + 4);
            const f32x4 b0 = *(const f32x4*)(sB + 32 * s + 8 * g), b1 = *(const f32x4*)(sB + 32 * s + 8 * g + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                fw[s][e] = from_f32<T>(x0[e] * bg0[e]);
                fw[s][4 + e] = from_f32<T>(x1[e] * bg1[e]);
                fu[s][e] = from_f32<T>(x0[e] * b0[e]);
                fu[s][4 + e] = from_f32<T>(x1[e] * b1[e]);
            }
        }
    }
    {
        T* wf = (T*)p.ws.Wf + (ci * HV + hv) * WS_W;
        for (int sp = 0; sp < 4; ++sp) {
            V8 frag;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int m = 2 * sp + half;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (s < ns) {
                        V8 ka;
#pragma unroll
                        for (int e = 0; e < 8; ++e) ka[e] = k_nat[(32 * s + 8 * g + e) * NP + 16 * m + c16];
                        acc = Mma<T>::run(ka, fw[s], acc);
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) frag[half * 4 + r] = from_f32<T>(acc[r]);
            }
            *(V8*)(wf + ((w * 4 + sp) * 64 + lane) * 8) = frag;
        }
        T* uf = (T*)p.ws.Uf + (ci * HV + hv) * WS_U;
        for (int n = 0; n < 8; ++n) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                if (s < ns) {
                    V8 vb;
#pragma unroll
                    for (int e = 0; e < 8; ++e) vb[e] = v_nat[(32 * s + 8 * g + e) * NP + 16 * n + c16];
                    acc = Mma<T>::run(fu[s], vb, acc);
                }
            }
            V4 o4;
#pragma unroll
            for (int r = 0; r < 4; ++r) o4[r] = from_f32<T>(acc[r]);
            *(V4*)(uf + ((n * 4 + w) * 64 + lane) * 4) = o4;
        }
    }
    // ---- k^T fragments for the state update (one copy per q/k head) ----
    if (hv % (HV / H) == 0) {
        T* ktf = (T*)p.ws.KTf + (ci * H + h) * WS_KT;
#pragma unroll
        for (int mm = 0; mm < 2; ++mm) {
            const int m = 2 * w + mm;
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                V8 frag;
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        frag[half * 4 + r] = k_nat[(32 * s + 16 * half + 4 * g + r) * NP + 16 * m + c16];
                *(V8*)(ktf + ((m * 2 + s) * 64 + lane) * 8) = frag;
            }
        }
    }
}

// ============================================================================================
// scan kernel
// ============================================================================================
template <typename T, int NV>
struct ScanFrags {
    typename Mma<T>::V8 wf[4], qf[4], kt[2][2], pf[2];
    typename Mma<T>::V4 uf[NV];
    f32x4 grow;
    float glast;
    int valid;
};

template <typename T, int NV>
__global__ __launch_bounds__(256) void gdn_chunk_scan_kernel(ChunkParams p) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    V8* sSb = (V8*)smem;                    // [4 s][NV][64] state as B operand (key tiles 2s, 2s+1)
    V4* sVn = (V4*)(sSb + 4 * NV * 64);     // [2 kind][2 s][NV][64][2 half] v_new as B operand (t-tiles 2s, 2s+1)

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    // Workgroups are dealt to the 8 XCDs round-robin by block index; keep all slabs of one
    // (sequence, head) on one XCD so that they share w / k^T / P / q through that XCD's L2.
    const int xcd = blockIdx.x & 7;
    const int64_t y = blockIdx.x >> 3;
    const int64_t inh = xcd + 8 * (y / p.nslab);
    const int slab = (int)(y % p.nslab);
    if (inh >= p.NH) return;
    const int H = p.H, HV = p.HV;
    const int64_t n = inh / HV;
    const int hv = (int)(inh % HV);
    const int h = hv / (HV / H);
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    const bool vfirst = p.flags & GDN_FLAG_STATE_V_FIRST;

    int64_t bos, len, boh;
    if (p.cu_seqlens) {
        bos = load_index(p.cu_seqlens, n, cu32);
        len = load_index(p.cu_seqlens, n + 1, cu32) - bos;
        boh = load_index(p.chunk_offsets, n, cu32);
    } else {
        bos = n * p.T;
        len = p.T;
        boh = n * p.NT;
    }
    const int64_t nt = (len + CH - 1) / CH;
    const int v0 = slab * NV * 16;          // first value column of this slab

    // ---- state: this wave owns key tiles 2w, 2w+1 (rows 32w .. 32w+31), C/D layout ----
    f32x4 S[2][NV];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
            if (p.h0) {
                const int kk = 32 * w + 16 * i + 4 * g, vc = v0 + 16 * nn + c16;
                const float* base = p.h0 + inh * 128 * 128;
                if (vfirst) s = *(const f32x4*)(base + vc * 128 + kk);
                else s = f32x4{base[kk * 128 + vc], base[(kk + 1) * 128 + vc], base[(kk + 2) * 128 + vc], base[(kk + 3) * 128 + vc]};
            }
            S[i][nn] = s;
        }

    const T* Wf = (const T*)p.ws.Wf;
    const T* Uf = (const T*)p.ws.Uf;
    const T* KTf = (const T*)p.ws.KTf;
    const T* Pf = (const T*)p.ws.Pf;
    const T* qg = (const T*)p.q;
    T* og = (T*)p.o;

    auto load_frags = [&](int64_t it, ScanFrags<T, NV>& f) {
        const int64_t ci = boh + it;
        const int64_t chv = ci * HV + hv;
        const int64_t tok0 = bos + it * CH;
        f.valid = (int)min((int64_t)CH, len - it * CH);
#pragma unroll
        for (int s = 0; s < 4; ++s) f.wf[s] = *(const V8*)(Wf + chv * WS_W + ((w * 4 + s) * 64 + lane) * 8);
        const int trow = 16 * w + c16;
        const T* qrow = qg + ((tok0 + trow) * H + h) * 128 + 4 * g;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            V4 a = {0, 0, 0, 0}, b = {0, 0, 0, 0};
            if (trow < f.valid && GDN_EXP != 2) {
                a = *(const V4*)(qrow + 32 * s);
                b = *(const V4*)(qrow + 32 * s + 16);
            }
            f.qf[s] = V8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int s = 0; s < 2; ++s)
                f.kt[i][s] = *(const V8*)(KTf + (ci * H + h) * WS_KT + (((2 * w + i) * 2 + s) * 64 + lane) * 8);
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            // P rows of t-tile w only reach t-tiles <= w: the second column pair exists for w >= 2
            if (s == 0 || w >= 2) f.pf[s] = *(const V8*)(Pf + chv * WS_P + ((w * 2 + s) * 64 + lane) * 8);
        }
#pragma unroll
        for (int nn = 0; nn < NV; ++nn)
            f.uf[nn] = *(const V4*)(Uf + chv * WS_U + (((v0 / 16 + nn) * 4 + w) * 64 + lane) * 4);
        f.grow = *(const f32x4*)(p.ws.G + chv * CH + 16 * w + 4 * g);
        f.glast = p.ws.G[chv * CH + CH - 1];
    };

    ScanFrags<T, NV> cur, nxt;
    if (nt > 0) load_frags(0, cur);
    nxt = cur;
    for (int64_t it = 0; it < nt; ++it) {
        if (it + 1 < nt && GDN_EXP != 4) load_frags(it + 1, nxt);
        // (a) publish the state of this chunk as bf16/f16 B-operand fragments
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            V8 f;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                f[r] = from_f32<T>(S[0][nn][r]);
                f[4 + r] = from_f32<T>(S[1][nn][r]);
            }
            sSb[(w * NV + nn) * 64 + lane] = f;
        }
        lds_barrier();
        // (b,c) w S and q S for t-tile w
        f32x4 accv[NV], acco[NV];
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            f32x4 av = {0.f, 0.f, 0.f, 0.f}, ao = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const V8 sb = sSb[(s * NV + nn) * 64 + lane];
                av = Mma<T>::run(cur.wf[s], sb, av);
                ao = Mma<T>::run(cur.qf[s], sb, ao);
            }
            accv[nn] = av;
            acco[nn] = ao;
        }
        // (d) v_new = u - w S; publish it plain (for the output) and decayed to the chunk end (for the state)
        const float glast = cur.glast;
        f32x4 dec, grow2;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            dec[r] = exp2f(glast - cur.grow[r]);
            grow2[r] = exp2f(cur.grow[r]);
        }
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            V4 plain, gated;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float vn = to_f32(cur.uf[nn][r]) - accv[nn][r];
                plain[r] = from_f32<T>(vn);
                gated[r] = from_f32<T>(vn * dec[r]);
            }
            sVn[(((0 * 2 + (w >> 1)) * NV + nn) * 64 + lane) * 2 + (w & 1)] = plain;
            sVn[(((1 * 2 + (w >> 1)) * NV + nn) * 64 + lane) * 2 + (w & 1)] = gated;
        }
        lds_barrier();
        // (e,f) state update and output
        const float gl2 = exp2f(glast);
        const V8* sVn8 = (const V8*)sVn;
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            const V8 vg0 = sVn8[((1 * 2 + 0) * NV + nn) * 64 + lane], vg1 = sVn8[((1 * 2 + 1) * NV + nn) * 64 + lane];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                f32x4 s = S[i][nn] * gl2;
                s = Mma<T>::run(cur.kt[i][0], vg0, s);
                s = Mma<T>::run(cur.kt[i][1], vg1, s);
                S[i][nn] = s;
            }
            f32x4 ao = acco[nn] * grow2;
            ao = Mma<T>::run(cur.pf[0], sVn8[((0 * 2 + 0) * NV + nn) * 64 + lane], ao);
            if (w >= 2) ao = Mma<T>::run(cur.pf[1], sVn8[((0 * 2 + 1) * NV + nn) * 64 + lane], ao);
            const int64_t tok0 = bos + it * CH;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = 16 * w + 4 * g + r;
#if GDN_EXP != 1
                if (t < cur.valid) og[((tok0 + t) * HV + hv) * 128 + v0 + 16 * nn + c16] = from_f32<T>(ao[r] * p.scale);
#else
                if (ao[r] == 12345.f) og[((tok0 + t) * HV + hv) * 128 + v0 + 16 * nn + c16] = from_f32<T>(ao[r] * p.scale);
#endif
            }
        }
        cur = nxt;
    }

    if (p.ht) {
        float* base = p.ht + inh * 128 * 128;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int nn = 0; nn < NV; ++nn) {
                const int kk = 32 * w + 16 * i + 4 * g, vc = v0 + 16 * nn + c16;
                if (vfirst) *(f32x4*)(base + vc * 128 + kk) = S[i][nn];
                else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) base[(kk + r) * 128 + vc] = S[i][nn][r];
                }
            }
    }
}

template <typename T, int NV>
static int launch_scan(const ChunkParams& p0, hipStream_t stream) {
    ChunkParams p = p0;
    p.nslab = 8 / NV;
    const size_t smem = (size_t)4 * NV * 64 * 16 + (size_t)2 * 2 * NV * 64 * 16;
    auto kern = gdn_chunk_scan_kernel<T, NV>;
    if (smem > 48 * 1024) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
            return check_launch("hipFuncSetAttribute(scan)");
    }
    const int64_t groups = (p.NH + 7) / 8;
    dim3 grid((unsigned)(groups * 8 * p.nslab)), block(256);
    hipLaunchKernelGGL(kern, grid, block, smem, stream, p);
    return check_launch("gdn_chunk_scan_kernel");
}

constexpr int STAGE_PREPARE = 1, STAGE_SCAN = 2;

template <typename T>
static int launch_chunk(const ChunkParams& p, int64_t num_chunks, int stages, hipStream_t stream) {
    if (stages & STAGE_PREPARE) {
        auto kern = gdn_chunk_prepare_kernel<T>;
        static bool attr_done = false;       // per instantiation
        if (!attr_done) {
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)PREP_SMEM) != hipSuccess)
                return check_launch("hipFuncSetAttribute(prepare)");
            attr_done = true;
        }
        dim3 grid((unsigned)num_chunks, (unsigned)p.HV), block(256);
        hipLaunchKernelGGL(kern, grid, block, PREP_SMEM, stream, p);
        int rc = check_launch("gdn_chunk_prepare_kernel");
        if (rc) return rc;
    }
    if (!(stages & STAGE_SCAN)) return GDN_OK;
    // widest value slab that still gives every CU a workgroup
    if (p.NH >= 256) return launch_scan<T, 8>(p, stream);
    if (p.NH * 2 >= 256) return launch_scan<T, 4>(p, stream);
    if (p.NH * 4 >= 256) return launch_scan<T, 2>(p, stream);
    return launch_scan<T, 1>(p, stream);
}

}  // namespace gdn

extern "C" size_t gdn_chunk_workspace_bytes(int64_t num_chunks, int64_t H, int64_t HV, int64_t K, int64_t V) {
    if (K != 128 || V != 128 || num_chunks < 0 || H < 1 || HV < 1) return 0;
    return gdn::ws_layout(num_chunks, H, HV, nullptr, nullptr);
}

static int chunk_entry(
    const char* who, int stages,
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    using namespace gdn;
    GDN_CHECK_ARG(q && k && v && g && beta && o, GDN_ERR_INVALID, "%s: q, k, v, g, beta, o must not be NULL", who);
    GDN_CHECK_ARG(B >= 1 && T >= 0 && H >= 1 && HV >= 1 && N >= 1, GDN_ERR_INVALID, "%s: non-positive dimension", who);
    GDN_CHECK_ARG(HV % H == 0, GDN_ERR_INVALID, "%s: HV=%lld not divisible by H=%lld", who, (long long)HV, (long long)H);
    GDN_CHECK_ARG(K == 128 && V == 128, GDN_ERR_UNSUPPORTED, "%s: only K = V = 128 is built (got K=%lld V=%lld)", who,
                  (long long)K, (long long)V);
    GDN_CHECK_ARG(qkv_dtype == GDN_DTYPE_BF16 || qkv_dtype == GDN_DTYPE_F16, GDN_ERR_UNSUPPORTED,
                  "%s: q/k/v must be bf16 or f16", who);
    GDN_CHECK_ARG(HV <= 65535, GDN_ERR_UNSUPPORTED, "%s: HV > 65535", who);
    if (cu_seqlens) {
        GDN_CHECK_ARG(B == 1, GDN_ERR_INVALID, "%s: with cu_seqlens B must be 1", who);
        GDN_CHECK_ARG(chunk_table && chunk_offsets, GDN_ERR_INVALID, "%s: packed input needs chunk_table and chunk_offsets", who);
    } else {
        GDN_CHECK_ARG(N == B, GDN_ERR_INVALID, "%s: without cu_seqlens N must equal B", who);
        GDN_CHECK_ARG(num_chunks == B * ((T + CH - 1) / CH), GDN_ERR_INVALID, "%s: num_chunks does not match B and T", who);
    }
    GDN_CHECK_ARG(((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0 && ((uintptr_t)h0 % 16) == 0 &&
                      ((uintptr_t)ht % 16) == 0 && ((uintptr_t)workspace % 256) == 0,
                  GDN_ERR_INVALID, "%s: q/k/v/h0/ht must be 16-byte and the workspace 256-byte aligned", who);
    if (T == 0 || num_chunks == 0) return GDN_OK;
    ChunkParams p;
    const size_t need = ws_layout(num_chunks, H, HV, (char*)workspace, &p.ws);
    GDN_CHECK_ARG(workspace && workspace_bytes >= need, GDN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who,
                  need, workspace_bytes);
    p.q = q; p.k = k; p.v = v; p.g = g; p.beta = beta; p.h0 = h0; p.ht = ht; p.o = o;
    p.cu_seqlens = cu_seqlens; p.chunk_table = chunk_table; p.chunk_offsets = chunk_offsets;
    p.T = T; p.H = (int)H; p.HV = (int)HV; p.N = N; p.NT = (T + CH - 1) / CH;
    p.scale = scale; p.gb_dtype = gb_dtype; p.flags = flags; p.nslab = 1; p.NH = N * HV;
    hipStream_t s = (hipStream_t)stream;
    return qkv_dtype == GDN_DTYPE_BF16 ? launch_chunk<bf16_t>(p, num_chunks, stages, s)
                                       : launch_chunk<f16_t>(p, num_chunks, stages, s);
}

#define GDN_CHUNK_ARGS                                                                          \
    const void *q, const void *k, const void *v, const void *g, const void *beta,               \
    const float *h0, float *ht, void *o,                                                        \
    const void *cu_seqlens, const void *chunk_table, const void *chunk_offsets,                 \
    void *workspace, size_t workspace_bytes,                                                    \
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,                          \
    int64_t N, int64_t num_chunks,                                                              \
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void *stream
#define GDN_CHUNK_PASS                                                                          \
    q, k, v, g, beta, h0, ht, o, cu_seqlens, chunk_table, chunk_offsets, workspace, workspace_bytes, \
    B, T, H, HV, K, V, N, num_chunks, scale, qkv_dtype, gb_dtype, flags, stream

extern "C" int gdn_chunk_fwd(GDN_CHUNK_ARGS) {
    return chunk_entry("gdn_chunk_fwd", gdn::STAGE_PREPARE | gdn::STAGE_SCAN, GDN_CHUNK_PASS);
}
extern "C" int gdn_chunk_fwd_prepare(GDN_CHUNK_ARGS) {
    return chunk_entry("gdn_chunk_fwd_prepare", gdn::STAGE_PREPARE, GDN_CHUNK_PASS);
}
extern "C" int gdn_chunk_fwd_scan(GDN_CHUNK_ARGS) {
    return chunk_entry("gdn_chunk_fwd_scan", gdn::STAGE_SCAN, GDN_CHUNK_PASS);
}
