// Chunk-parallel stage of the chunked prefill: one workgroup per (chunk, v-head) computes
// what does not depend on the running state and is not a plain copy of the inputs:
//   G = cumsum(g)/ln2,  L = beta*(K K^T)*2^(G_i-G_j) (i>j),  X = (I+L)^-1 in fp32 (16x16 forward
//   substitution on the diagonal blocks, fp32-MFMA block merges),  Xb = X diag(beta),
//   P = scale*tril(q k^T * 2^(G_i-G_j)),  and the per-token gate tables.
// Xb and P are written in the exact register order ("fragments") in which the scan kernel
// feeds them to the matrix cores; the scan forms v_new = Xb (v - 2^G (k S)) itself from the
// raw k and v, so neither w = Xb 2^G k nor u = Xb v is ever materialised.
#include "gdn_chunk_common.h"

namespace gdn {

constexpr int NP = 128 + 8;     // pitch (elements) of the staged 64x128 tiles: 272 B rows, conflict-free 16 B reads
constexpr int LP = 68;          // pitch (floats) of the 64x64 fp32 matrices
constexpr size_t PREP_SMEM = 3 * CH * NP * 2 + 2 * CH * 4;     // 52 736 B: three workgroups per CU

template <typename T>
__global__ __launch_bounds__(256) void gdn_chunk_prepare_kernel(ChunkParams p) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    T* k_nat = (T*)smem;                        // [64][NP] keys, token-major
    T* q_nat = k_nat + CH * NP;                 // [64][NP] queries; the region is reused for X below
    float* sL = (float*)(q_nat + CH * NP);      // [64][LP] L (strictly lower); 64*68*4 == 64*136*2 bytes
    float* sX = (float*)q_nat;                  // [64][LP] (I+L)^-1, same bytes as q_nat
    float* sG = sL + CH * LP;                   // [64] cumulative gate (log2)
    float* sB = sG + CH;                        // [64] beta

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

    // ---- stage k, q (rows past the end of the sequence are zero) ----
    const T* kg = (const T*)p.k + (tok0 * H + h) * 128;
    const T* qg = (const T*)p.q + (tok0 * H + h) * 128;
    u32x4 rk[4], rq[4];
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int row = ps * 16 + (tid >> 4), col = (tid & 15) * 8;
        const u32x4 z = {0u, 0u, 0u, 0u};
        rk[ps] = rq[ps] = z;
        if (row < valid) {
            rk[ps] = *(const u32x4*)(kg + (int64_t)row * H * 128 + col);
            rq[ps] = *(const u32x4*)(qg + (int64_t)row * H * 128 + col);
        }
    }
    char* rec = p.ws.Rec + (ci * HV + hv) * REC_BYTES;
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
        float* tab = (float*)(rec + REC_TAB);
        tab[TAB_DEC + lane] = fast_exp2(xl - x);
        tab[TAB_SG + lane] = p.scale * ex;
        tab[TAB_EG + lane] = ex;
        if (lane == 63) tab[TAB_GLAST] = x;
    }
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int row = ps * 16 + (tid >> 4), col = (tid & 15) * 8;
        *(u32x4*)(k_nat + row * NP + col) = rk[ps];
        *(u32x4*)(q_nat + row * NP + col) = rq[ps];
    }
    __syncthreads();

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
        T* pf = (T*)(rec + REC_P);
        for (int sp = 0; sp < 2; ++sp) {
            if (tt < 2 && sp == 1) continue;        // identically zero, not stored
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
            *(V8*)(pf + (p_slot(tt, sp) * 64 + lane) * 8) = frag;
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
#pragma unroll
        for (int r = 0; r < 4; ++r) tmp2[(16 * a + 4 * g + r) * LP + 16 * b + c16] = y[r];
        __syncthreads();
        f32x4 z = mm16_f32(sX + (32 + 16 * a) * LP + 32, LP, tmp2 + 16 * b, LP, 8, c16, g);
#pragma unroll
        for (int r = 0; r < 4; ++r) sX[(32 + 16 * a + 4 * g + r) * LP + 16 * b + c16] = -z[r];
    }
    __syncthreads();
    // ---- Xb = X diag(beta) rows of t-tile w as A-operand fragments ----
    {
        T* xf = (T*)(rec + REC_X);
        const int ns = (w >= 2) ? 2 : 1;         // X is lower triangular: columns >= 32 matter only for rows >= 32
        for (int sp = 0; sp < ns; ++sp) {
            const float* xr = sX + (16 * w + c16) * LP + 32 * sp + 4 * g;
            const f32x4 x0 = *(const f32x4*)xr, x1 = *(const f32x4*)(xr + 16);
            const f32x4 b0 = *(const f32x4*)(sB + 32 * sp + 4 * g), b1 = *(const f32x4*)(sB + 32 * sp + 16 + 4 * g);
            V8 frag;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                frag[e] = from_f32<T>(x0[e] * b0[e]);
                frag[4 + e] = from_f32<T>(x1[e] * b1[e]);
            }
            *(V8*)(xf + (p_slot(w, sp) * 64 + lane) * 8) = frag;
        }
    }
}

template <typename T>
int launch_prepare(const ChunkParams& p, int64_t num_chunks, hipStream_t stream) {
    auto kern = gdn_chunk_prepare_kernel<T>;
    static bool attr_done = false;       // per instantiation
    if (!attr_done) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)PREP_SMEM) != hipSuccess)
            return check_launch("hipFuncSetAttribute(prepare)");
        attr_done = true;
    }
    dim3 grid((unsigned)num_chunks, (unsigned)p.HV), block(256);
    hipLaunchKernelGGL(kern, grid, block, PREP_SMEM, stream, p);
    return check_launch("gdn_chunk_prepare_kernel");
}
template int launch_prepare<bf16_t>(const ChunkParams&, int64_t, hipStream_t);
template int launch_prepare<f16_t>(const ChunkParams&, int64_t, hipStream_t);

}  // namespace gdn
