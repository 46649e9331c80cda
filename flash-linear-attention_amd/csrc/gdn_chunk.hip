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
#include <type_traits>

namespace gdn {

constexpr int CH = 64;                       // chunk length
constexpr float RCP_LN2_F = 1.4426950216f;   // fla/ops/utils/constant.py:10

typedef bf16x4 __attribute__((address_space(3)))* lds_bf16x4_ptr;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef s16x4 __attribute__((address_space(3)))* lds_s16x4_ptr;

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    typedef bf16x8 V8;
    typedef bf16x4 V4;
    static __device__ __forceinline__ f32x4 run(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    // LDS transpose read: the 16 lanes of a group each pass the address of 4 consecutive
    // elements; lane L receives element L%4 of the runs addressed by lanes L/4, L/4+4, L/4+8, L/4+12.
    static __device__ __forceinline__ V4 tr_read(const bf16_t* p) {
        return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)p);
    }
};
template <> struct Mma<f16_t> {
    typedef f16x8 V8;
    typedef f16x4 V4;
    static __device__ __forceinline__ f32x4 run(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ V4 tr_read(const f16_t* p) {
        return __builtin_bit_cast(f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p));
    }
};

template <typename V8, typename V4>
__device__ __forceinline__ V8 join(V4 a, V4 b) {
    return V8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
}

// 2^x as a single v_exp_f32 (results below 2^-126 flush to zero, which is what a decay wants)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Per-chunk workspace written by the prepare kernel (element counts for K = V = 128):
//   Tab fp32 [NC][HV][192]                  [0..63] 2^(G_last-G_t), [64..127] scale*2^G_t, [128] G_last (log2 units)
//   Wf  T    [NC][HV][4 tt][4 s][64][8]     w rows of t-tile tt, key tiles (2s, 2s+1)
//   Uf  T    [NC][HV][8 n ][4 tt][64][4]    u, C/D layout of tile (t-tile tt, value tile n)
//   Pf  T    [NC][HV][4 tt][2 s][64][8]     scale*P rows of t-tile tt, t-tiles (2s, 2s+1) as columns
//   KTf T    [NC][H ][8 m ][2 s][64][8]     k^T rows of key tile m, t-tiles (2s, 2s+1)
//   Qf  T    [NC][H ][4 tt][4 s][64][8]     q rows of t-tile tt, key tiles (2s, 2s+1)
struct ChunkWs {
    float* Tab;
    void* Wf;
    void* Uf;
    void* Pf;
    void* KTf;
    void* Qf;
};
constexpr int64_t WS_TAB = 192, WS_W = 8192, WS_U = 8192, WS_P = 4096, WS_KT = 8192, WS_Q = 8192;   // elements per (chunk, head)

static size_t ws_align(size_t x) { return (x + 255) & ~(size_t)255; }

static size_t ws_layout(int64_t NC, int64_t H, int64_t HV, char* base, ChunkWs* ws) {
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += ws_align(bytes); return base ? (void*)(base + o) : nullptr; };
    void* Tab = take((size_t)NC * HV * WS_TAB * 4);
    void* Wf = take((size_t)NC * HV * WS_W * 2);
    void* Uf = take((size_t)NC * HV * WS_U * 2);
    void* Pf = take((size_t)NC * HV * WS_P * 2);
    void* KTf = take((size_t)NC * H * WS_KT * 2);
    void* Qf = take((size_t)NC * H * WS_Q * 2);
    if (ws) { ws->Tab = (float*)Tab; ws->Wf = Wf; ws->Uf = Uf; ws->Pf = Pf; ws->KTf = KTf; ws->Qf = Qf; }
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
// the vector-memory counter, which would serialise the global prefetch of later chunks
// behind every barrier of the current one.
#ifndef GDN_EXP
#define GDN_EXP 0
#endif
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 8-byte global store issued from inline assembly.  The compiler's wait-count bookkeeping
// does not see it, so the prefetched loads of the scan loop stay the only operations it
// counts and it can wait for "all but the newest N loads" instead of draining the queue
// (loads and stores share one hardware counter, and once both are pending the compiler
// falls back to waiting for everything).  The extra, uncounted stores only make the
// hardware counter larger than the compiler assumes, i.e. its waits err on the late side.
__device__ __forceinline__ void store_b64_uncounted(void* ptr, u32x2 data) {
    asm volatile("global_store_dwordx2 %0, %1, off" : : "v"(ptr), "v"(data) : "memory");
}

// 16x16 product of fp32 matrices held in LDS on the fp32 matrix cores:
// C = A[16 x 4*nk] * B[4*nk x 16]; result in C/D layout.
__device__ __forceinline__ f32x4 mm16_f32(const float* A, int lda, const float* B, int ldb, int nk, int c16, int g) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
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
constexpr size_t PREP_SMEM = 3 * CH * NP * 2 + 3 * CH * 4;     // 52 992 B: three workgroups per CU

// Transposed MFMA operand from a token-major tile: lane (c16, g) gets column fb + c16 of the
// 8 rows r0 .. r0+7 (two transpose reads of 4 rows each).
template <typename T>
__device__ __forceinline__ typename Mma<T>::V8 tr_frag8(const T* tile, int r0, int fb, int c16) {
    const T* a = tile + (r0 + (c16 >> 2)) * NP + fb + 4 * (c16 & 3);
    return join<typename Mma<T>::V8>(Mma<T>::tr_read(a), Mma<T>::tr_read(a + 4 * NP));
}
// Same for two separate groups of 4 rows starting at ra and rb.
template <typename T>
__device__ __forceinline__ typename Mma<T>::V8 tr_frag44(const T* tile, int ra, int rb, int fb, int c16) {
    const int o = (c16 >> 2) * NP + fb + 4 * (c16 & 3);
    return join<typename Mma<T>::V8>(Mma<T>::tr_read(tile + ra * NP + o), Mma<T>::tr_read(tile + rb * NP + o));
}

template <typename T>
__global__ __launch_bounds__(256) void gdn_chunk_prepare_kernel(ChunkParams p) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    T* k_nat = (T*)smem;                        // [64][NP] keys, token-major
    T* q_nat = k_nat + CH * NP;                 // [64][NP] queries; the region is reused for X below
    T* v_nat = q_nat + CH * NP;                 // [64][NP] values; staged only after the solve (same bytes as L)
    float* sL = (float*)v_nat;                  // [64][LP] L (strictly lower); 64*68*4 == 64*136*2 bytes
    float* sX = (float*)q_nat;                  // [64][LP] (I+L)^-1, same bytes as q_nat
    float* sG = (float*)(v_nat + CH * NP);      // [64] cumulative gate (log2)
    float* sB = sG + CH;                        // [64] beta
    float* sBG = sB + CH;                       // [64] beta * 2^G

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    const int64_t ci = blockIdx.x;
    const int hv = blockIdx.y;
    const int H = p.H, HV = p.HV;
    const int h = hv / (HV / H);
    const bool first_of_group = hv % (HV / H) == 0;      // writes the per-q/k-head fragments
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
        const float xl = __shfl(x, 63, 64);      // rows past the end carry the last valid sum
        const float ex = fast_exp2(x);
        sG[lane] = x;
        sB[lane] = b;
        sBG[lane] = b * ex;
        float* tab = p.ws.Tab + (ci * HV + hv) * WS_TAB;
        tab[lane] = fast_exp2(xl - x);
        tab[64 + lane] = p.scale * ex;
        if (lane == 63) tab[128] = x;
    }
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int row = ps * 16 + (tid >> 4), col = (tid & 15) * 8;
        *(u32x4*)(k_nat + row * NP + col) = rk[ps];
        *(u32x4*)(q_nat + row * NP + col) = rq[ps];
    }
    __syncthreads();
#if GDN_EXP == 5
    return;
#endif

    // ---- L tiles of row-tile w (K K^T, gated, beta-scaled, strictly lower) ----
    {
        V8 ka[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) ka[s] = *(const V8*)(k_nat + (16 * w + c16) * NP + 32 * s + 8 * g);
        const f32x4 gi = *(const f32x4*)(sG + 16 * w + 4 * g), bi = *(const f32x4*)(sB + 16 * w + 4 * g);
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
                sL[i * LP + j] = (i > j) ? bi[r] * acc[r] * fast_exp2(gi[r] - gj) : 0.f;
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
        for (int sp = 0; sp < 2; ++sp) {
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
                const f32x4 gj = *(const f32x4*)(sG + 16 * tj + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = 16 * tj + 4 * g + r;
                    const float val = (t >= j) ? p.scale * acc[r] * fast_exp2(gt - gj[r]) : 0.f;
                    frag[half * 4 + r] = from_f32<T>(val);
                }
            }
            *(V8*)(pf + ((tt * 2 + sp) * 64 + lane) * 8) = frag;
        }
        // q rows of t-tile tt as A operands over key tiles (2s, 2s+1), one copy per q/k head
        if (first_of_group) {
            T* qf = (T*)p.ws.Qf + (ci * H + h) * WS_Q;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const T* src = q_nat + (16 * tt + c16) * NP + 32 * s + 4 * g;
                *(V8*)(qf + ((tt * 4 + s) * 64 + lane) * 8) = join<V8>(*(const V4*)src, *(const V4*)(src + 16));
            }
        }
    }
    __syncthreads();     // L complete; q_nat is dead from here on and becomes X
#if GDN_EXP == 6
    return;
#endif

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
#pragma unroll
        for (int r = 0; r < 4; ++r) tmp2[(16 * a + 4 * g + r) * LP + 16 * b + c16] = y[r];
        __syncthreads();
        f32x4 z = mm16_f32(sX + (32 + 16 * a) * LP + 32, LP, tmp2 + 16 * b, LP, 8, c16, g);
#pragma unroll
        for (int r = 0; r < 4; ++r) sX[(32 + 16 * a + 4 * g + r) * LP + 16 * b + c16] = -z[r];
    }
    __syncthreads();
    // L is dead: its bytes now take the value tile, which has been waiting in registers
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int row = ps * 16 + (tid >> 4), col = (tid & 15) * 8;
        *(u32x4*)(v_nat + row * NP + col) = rv[ps];
    }
    __syncthreads();

#if GDN_EXP == 7
    return;
#endif
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
#pragma unroll
        for (int sp = 0; sp < 4; ++sp) {
            V8 frag;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int m = 2 * sp + half;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < 2; ++s)
                    if (s < ns) acc = Mma<T>::run(tr_frag8<T>(k_nat, 32 * s + 8 * g, 16 * m, c16), fw[s], acc);
#pragma unroll
                for (int r = 0; r < 4; ++r) frag[half * 4 + r] = from_f32<T>(acc[r]);
            }
            *(V8*)(wf + ((w * 4 + sp) * 64 + lane) * 8) = frag;
        }
        T* uf = (T*)p.ws.Uf + (ci * HV + hv) * WS_U;
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; ++s)
                if (s < ns) acc = Mma<T>::run(fu[s], tr_frag8<T>(v_nat, 32 * s + 8 * g, 16 * n, c16), acc);
            V4 o4;
#pragma unroll
            for (int r = 0; r < 4; ++r) o4[r] = from_f32<T>(acc[r]);
            *(V4*)(uf + ((n * 4 + w) * 64 + lane) * 4) = o4;
        }
    }
    // ---- k^T fragments for the state update (one copy per q/k head) ----
    if (first_of_group) {
        T* ktf = (T*)p.ws.KTf + (ci * H + h) * WS_KT;
#pragma unroll
        for (int mm = 0; mm < 2; ++mm) {
            const int m = 2 * w + mm;
#pragma unroll
            for (int s = 0; s < 2; ++s)
                *(V8*)(ktf + ((m * 2 + s) * 64 + lane) * 8) = tr_frag44<T>(k_nat, 32 * s + 4 * g, 32 * s + 16 + 4 * g, 16 * m, c16);
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
    f32x4 dec;          // 2^(G_last-G_t) for the 4 rows of this lane's C/D fragment
    float gam;          // scale*2^G_t for the column of this lane's transposed output fragment
    float glast;        // G_last in log2 units
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

    // Make the initial state arrive before the prefetch queue is started: a wait for these
    // registers inside the loop (their first use) would be executed on every trip and would
    // drain the prefetched loads with it.
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) asm volatile("" : "+v"(S[i][nn]) : : "memory");

    const T* Wf = (const T*)p.ws.Wf;
    const T* Uf = (const T*)p.ws.Uf;
    const T* KTf = (const T*)p.ws.KTf;
    const T* Pf = (const T*)p.ws.Pf;
    const T* Qf = (const T*)p.ws.Qf;
    T* og = (T*)p.o;

    // All loads are unconditional and there is no data-dependent control flow around memory
    // operations in the main loop: the compiler can then count outstanding loads exactly and
    // wait only for the buffer it is about to use, instead of draining the queue.
    auto load_a = [&](int64_t it, ScanFrags<T, NV>& f) {        // operands of the first half of a step
        const int64_t ci = boh + it;
        const int64_t chv = ci * HV + hv, ch = ci * H + h;
#pragma unroll
        for (int s = 0; s < 4; ++s) f.wf[s] = *(const V8*)(Wf + chv * WS_W + ((w * 4 + s) * 64 + lane) * 8);
#pragma unroll
        for (int s = 0; s < 4; ++s) f.qf[s] = *(const V8*)(Qf + ch * WS_Q + ((w * 4 + s) * 64 + lane) * 8);
    };
    auto load_b = [&](int64_t it, ScanFrags<T, NV>& f) {        // everything else
        const int64_t ci = boh + it;
        const int64_t chv = ci * HV + hv, ch = ci * H + h;
        f.valid = (int)min((int64_t)CH, len - it * CH);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int s = 0; s < 2; ++s)
                f.kt[i][s] = *(const V8*)(KTf + ch * WS_KT + (((2 * w + i) * 2 + s) * 64 + lane) * 8);
#pragma unroll
        for (int s = 0; s < 2; ++s) f.pf[s] = *(const V8*)(Pf + chv * WS_P + ((w * 2 + s) * 64 + lane) * 8);
#pragma unroll
        for (int nn = 0; nn < NV; ++nn)
            f.uf[nn] = *(const V4*)(Uf + chv * WS_U + (((v0 / 16 + nn) * 4 + w) * 64 + lane) * 4);
        const float* tab = p.ws.Tab + chv * WS_TAB;
        f.dec = *(const f32x4*)(tab + 16 * w + 4 * g);
        f.gam = tab[64 + 16 * w + c16];
        f.glast = tab[128];
    };

    // The registers hold Shat = S / Gamma with one scalar Gamma = 2^lg per workgroup, so the
    // decay of the whole state by 2^G_last per chunk costs nothing: products with S are
    // rescaled by Gamma (folded into multiplies that exist anyway) and the update is divided
    // by the new Gamma (folded into the decay factors of v_new).  When Gamma gets small the
    // state is rescaled once and Gamma restarts at 1.  f16 operands have too little range for
    // Shat, so there the state is rescaled on every chunk.
    constexpr float LG_MIN = std::is_same<T, bf16_t>::value ? -60.f : 1.f;
    float lg = 0.f;                                              // log2 Gamma

    // `f` holds the chunk being processed; `fr` is the buffer consumed one step earlier, which is
    // refilled with chunk `refill` while this step computes (its loads are interleaved with the
    // matrix instructions so that the memory pipeline never sees a burst).
    auto step = [&](int64_t it, ScanFrags<T, NV>& f, ScanFrags<T, NV>& fr, int64_t refill, auto masked) {
        // (a) publish the state at the start of this chunk as bf16/f16 B-operand fragments
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            V8 sb;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sb[r] = from_f32<T>(S[0][nn][r]);
                sb[4 + r] = from_f32<T>(S[1][nn][r]);
            }
            sSb[(w * NV + nn) * 64 + lane] = sb;
        }
        const float gamma = fast_exp2(lg);
        const float lg_try = lg + f.glast;
        const bool lazy = lg_try >= LG_MIN;                      // same value in every lane of the workgroup
        const float vscale = lazy ? fast_exp2(-lg_try) : 1.f;
        const f32x4 dec = f.dec * vscale;
        const float ogam = f.gam * gamma;
        lds_barrier();
        // (b,c) w S (rows of t-tile w) and (q S)^T (columns of t-tile w)
        f32x4 acco[NV];
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            f32x4 av = {0.f, 0.f, 0.f, 0.f}, ao = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const V8 sb = sSb[(s * NV + nn) * 64 + lane];
                av = Mma<T>::run(f.wf[s], sb, av);
                ao = Mma<T>::run(sb, f.qf[s], ao);      // operands swapped: result is the transposed tile
            }
            acco[nn] = ao * ogam;
            // (d) v_new = u - w S; publish it plain (for the output) and decayed to the chunk end (for the state)
            V4 plain, gated;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float vn = to_f32(f.uf[nn][r]) - gamma * av[r];
                plain[r] = from_f32<T>(vn);
                gated[r] = from_f32<T>(vn * dec[r]);
            }
            sVn[(((0 * 2 + (w >> 1)) * NV + nn) * 64 + lane) * 2 + (w & 1)] = plain;
            sVn[(((1 * 2 + (w >> 1)) * NV + nn) * 64 + lane) * 2 + (w & 1)] = gated;
        }
        if (!decltype(masked)::value) {
            load_a(refill, fr);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                __builtin_amdgcn_sched_group_barrier(0x008, NV, 0);      // NV matrix instructions
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);       // then one global load
            }
        }
        if (!lazy) {
            const float fold = fast_exp2(lg_try);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int nn = 0; nn < NV; ++nn) S[i][nn] *= fold;
        }
        lg = lazy ? lg_try : 0.f;
        lds_barrier();
        // (e,f) state update and output
        const V8* sVn8 = (const V8*)sVn;
        const int trow = 16 * w + c16;
        T* orow = og + ((bos + it * CH + trow) * HV + hv) * 128 + v0 + 4 * g;
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            const V8 vg0 = sVn8[((1 * 2 + 0) * NV + nn) * 64 + lane], vg1 = sVn8[((1 * 2 + 1) * NV + nn) * 64 + lane];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                f32x4 s = S[i][nn];
                s = Mma<T>::run(f.kt[i][0], vg0, s);
                s = Mma<T>::run(f.kt[i][1], vg1, s);
                S[i][nn] = s;
            }
            // P rows of t-tile w reach t-tiles <= w only; the fragments above the diagonal are zero
            f32x4 ao = Mma<T>::run(sVn8[((0 * 2 + 0) * NV + nn) * 64 + lane], f.pf[0], acco[nn]);
            ao = Mma<T>::run(sVn8[((0 * 2 + 1) * NV + nn) * 64 + lane], f.pf[1], ao);
            // transposed tile: this lane holds 4 consecutive value columns of token row trow
            V4 o4;
#pragma unroll
            for (int r = 0; r < 4; ++r) o4[r] = from_f32<T>(ao[r]);
            if (!decltype(masked)::value) store_b64_uncounted(orow + 16 * nn, __builtin_bit_cast(u32x2, o4));
            else if (trow < f.valid) *(V4*)(orow + 16 * nn) = o4;
        }
        if (!decltype(masked)::value) {
            load_b(refill, fr);
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                __builtin_amdgcn_sched_group_barrier(0x008, NV, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
            }
        }
    };
    std::integral_constant<bool, false> full_chunk;
    std::integral_constant<bool, true> tail_chunk;

    // NB fragment buffers in rotation: step `it` computes from buffer it%NB and refills buffer
    // (it-1)%NB (consumed in the previous step) with chunk it+NB-1, so every load has NB-2 full
    // steps to arrive.  A wave can have 63 loads in flight, 18 per buffer, hence NB = 4.
    // Refills past the end re-read the last chunk and are never used.
    constexpr int NB = NV >= 8 ? 3 : 4;          // the widest slab has no registers to spare and is compute-bound anyway
    ScanFrags<T, NV> fb[NB];
    const int64_t last = nt - 1;
    const int64_t nfast = (len / CH) / NB * NB;     // chunks handled NB at a time; all of them are full
    if (nt > 0) {
        // compiler fences keep the groups in issue order, as inside the loop: the waits in the
        // loop are sized for the entry path too
#pragma unroll
        for (int j = 0; j < NB - 1; ++j) {
            load_a(min((int64_t)j, last), fb[j]);
            asm volatile("" ::: "memory");
            load_b(min((int64_t)j, last), fb[j]);
            asm volatile("" ::: "memory");
        }
    }
    for (int64_t it = 0; it < nfast; it += NB) {
#pragma unroll
        for (int j = 0; j < NB; ++j) step(it + j, fb[j], fb[(j + NB - 1) % NB], min(it + j + NB - 1, last), full_chunk);
    }
    // at most NB chunks remain (NB-1 full ones and a ragged tail): buffers 0..NB-2 already hold
    // the first of them
    if (nfast + NB - 1 < nt) {
        load_a(nfast + NB - 1, fb[NB - 1]);
        load_b(nfast + NB - 1, fb[NB - 1]);
    }
#pragma unroll
    for (int j = 0; j < NB; ++j)
        if (nfast + j < nt) step(nfast + j, fb[j], fb[j], 0, tail_chunk);

    // back to the true state
    {
        const float gamma = fast_exp2(lg);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int nn = 0; nn < NV; ++nn) S[i][nn] *= gamma;
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
