// Chunk-parallel stage of the chunked prefill: one workgroup per (chunk, q/k head) computes
// what does not depend on the running state and is not a plain copy of the inputs, for every
// value head of that q/k head:
//   G = cumsum(g)/ln2,  L = beta*(K K^T)*2^(G_i-G_j) (i>j),  X = (I+L)^-1 in fp32 (16x16 forward
//   substitution on the diagonal blocks, fp32-MFMA block merges),  Xb = X diag(beta),
//   P = scale*tril(q k^T * 2^(G_i-G_j)),  and the per-token gate tables.
// Optional prologues of the reference are folded in: the gate and beta activations, and the l2
// normalisation of q and k as per-row factors 1/|k_t|, 1/|q_t| on L, P and the tables (so the
// sequential stage reads q and k exactly as the caller gave them).
// The raw products K K^T and q K^T are formed once and stay in registers; the value heads differ
// only in their gates.  Xb and P are written in the exact register order ("fragments") in which
// the scan kernel feeds them to the matrix cores; the scan forms v_new = Xb (v - 2^G (k S)) itself
// from the raw k and v, so neither w = Xb 2^G k nor u = Xb v is ever materialised.
#include "gdn_chunk_common.h"

namespace gdn {

constexpr int NP = 128 + 8;     // pitch (elements) of the staged 64x128 tiles: 272 B rows, conflict-free 16 B reads
constexpr int LP = 68;          // pitch (floats) of the 64x64 fp32 matrices
// two tiles (k then L, q then X), the transposed diagonal blocks of L, the row factors of k and q, and gates + beta
// of every value head of the group
inline size_t prep_smem(int group) { return 2 * CH * NP * 2 + 4 * 16 * 16 * 4 + 3 * CH * 4 + (size_t)group * 2 * CH * 4; }

template <typename T>
__global__ __launch_bounds__(256, 4) void gdn_chunk_prepare_kernel(ChunkParams p) {
    typedef typename Mma<T>::V8 V8;
    extern __shared__ __align__(16) char smem[];
    T* k_nat = (T*)smem;                        // [64][NP] keys, token-major; reused for L once the raw products exist
    T* q_nat = k_nat + CH * NP;                 // [64][NP] queries; reused for X
    float* sL = (float*)k_nat;                  // [64][LP] L (strictly lower); 64*68*4 == 64*136*2 bytes
    float* sX = (float*)q_nat;                  // [64][LP] (I+L)^-1
    float* sLd = (float*)(q_nat + CH * NP);     // [4][16 j][16 i] diagonal blocks of L, transposed (column j contiguous)
    float* sRN = sLd + 4 * 256;                 // [3][64] 1/|k_t|, 1/|q_t| (ones unless the rows are to be normalised), |k_t|^2 as given
    float* sGB = sRN + 3 * CH;                  // [group][2][64] cumulative gate (log2), beta

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    // heads vary fastest over the workgroups: those that run at the same time then read whole token rows
    // (all heads of a token are contiguous in memory) instead of one 256-byte piece of every row
    const int H = p.H, HV = p.HV;
    const int64_t ci = blockIdx.x / H;
    const int h = (int)(blockIdx.x % H);
    const int G = HV / H;
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

    // q is needed for its row norms (l2 normalisation) and for P, when P is asked for
    const bool l2 = p.flags & GDN_FLAG_QK_L2NORM;
    const bool want_P = p.want_P != 0, need_q = l2 || want_P;
    // ---- all global loads first: the gate inputs of value head w of the group, then the k, q rows ----
    float rg = 0.f, rb = 0.f;
    if (w < G && lane < valid) {
        rg = p.g ? load_scalar(p.g, (tok0 + lane) * HV + h * G + w, p.gb_dtype) : 0.f;      // (no gate: the plain delta rule)
        rb = load_scalar(p.beta, (tok0 + lane) * HV + h * G + w, p.gb_dtype);
    }
    // ---- k (and q) rows, 128 key features at a time (K <= 128: one round): into LDS, their squared norms, and the raw
    // products, which stay in registers: K K^T tiles (row-tile w, column-tiles <= w) and the transposed q K^T tiles
    // of query tile tt = 3 - w (key tiles <= tt).  Rows past the end of the sequence and key features past K are zero.
    const int tt = 3 - w;
    f32x4 kk[4], qk[4];
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) kk[tj] = qk[tj] = f32x4{0.f, 0.f, 0.f, 0.f};
    {
        const int K = p.K;
        const T* kg = (const T*)p.k + (tok0 * H + h) * K;
        const T* qg = (const T*)p.q + (tok0 * H + h) * K;
        float sk[4] = {0.f, 0.f, 0.f, 0.f}, sq[4] = {0.f, 0.f, 0.f, 0.f};
        for (int k0 = 0; k0 < K; k0 += 128) {
            if (k0) __syncthreads();                 // the products of the previous round have read the tiles
            u32x4 rk[4], rq[4];
#pragma unroll
            for (int ps = 0; ps < 4; ++ps) {
                const int row = ps * 16 + (tid >> 4), col = k0 + (tid & 15) * 8;
                const u32x4 z = {0u, 0u, 0u, 0u};
                rk[ps] = rq[ps] = z;
                if (row < valid && col < K) {
                    rk[ps] = *(const u32x4*)(kg + (int64_t)row * H * K + col);
                    if (need_q) rq[ps] = *(const u32x4*)(qg + (int64_t)row * H * K + col);
                }
            }
#pragma unroll
            for (int ps = 0; ps < 4; ++ps) {
                const int row = ps * 16 + (tid >> 4), col = (tid & 15) * 8;
                *(u32x4*)(k_nat + row * NP + col) = rk[ps];
                if (want_P) *(u32x4*)(q_nat + row * NP + col) = rq[ps];
                // l2 normalisation is applied as per-row factors: 16 lanes hold one row
                if (l2) {
                    const V8 k8 = __builtin_bit_cast(V8, rk[ps]), q8 = __builtin_bit_cast(V8, rq[ps]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) { const float a = to_f32(k8[e]), b = to_f32(q8[e]); sk[ps] += a * a; sq[ps] += b * b; }
                }
            }
            if (k0 + 128 >= K) {
#pragma unroll
                for (int ps = 0; ps < 4; ++ps) {
                    float a = sk[ps], b = sq[ps];
                    if (l2) {
#pragma unroll
                        for (int off = 1; off < 16; off <<= 1) { a += __shfl_xor(a, off, 64); b += __shfl_xor(b, off, 64); }
                    }
                    if ((tid & 15) == 0) {
                        const int row = ps * 16 + (tid >> 4);
                        sRN[row] = l2 ? rsqrtf(a + 1e-6f) : 1.f;
                        sRN[CH + row] = l2 ? rsqrtf(b + 1e-6f) : 1.f;
                    }
                }
            }
            __syncthreads();
            V8 ka[4], qb[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                ka[s] = *(const V8*)(k_nat + (16 * w + c16) * NP + 32 * s + 8 * g);
                if (want_P) qb[s] = *(const V8*)(q_nat + (16 * tt + c16) * NP + 32 * s + 8 * g);
            }
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                if (tj <= w || (want_P && tj <= tt)) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const V8 kb = *(const V8*)(k_nat + (16 * tj + c16) * NP + 32 * s + 8 * g);
                        if (tj <= w) kk[tj] = Mma<T>::run(ka[s], kb, kk[tj]);          // rows: tokens of tile w, column: token 16tj + c16
                        if (want_P && tj <= tt) qk[tj] = Mma<T>::run(kb, qb[s], qk[tj]);         // rows: key tokens of tile tj, column: query token 16tt + c16
                    }
                }
            }
        }
    }
    // ---- gates of every value head of the group: inclusive scan over the chunk, one token per lane ----
    for (int m = w; m < G; m += 4) {
        const int hv = h * G + m;
        float x = rg, b = rb;
        if (m >= 4) {                            // beyond the four fetched up front
            x = b = 0.f;
            if (lane < valid) {
                x = p.g ? load_scalar(p.g, (tok0 + lane) * HV + hv, p.gb_dtype) : 0.f;
                b = load_scalar(p.beta, (tok0 + lane) * HV + hv, p.gb_dtype);
            }
        }
        if (lane < valid) {                      // optional activations of the raw gate / beta inputs
            if (p.A_log && p.g) x = -__expf(p.A_log[hv]) * softplus_f(x + (p.dt_bias ? p.dt_bias[hv] : 0.f));
            if (p.flags & GDN_FLAG_BETA_SIGMOID) b = sigmoid_f(b) * ((p.flags & GDN_FLAG_NEG_EIGVAL) ? 2.f : 1.f);
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float y = __shfl_up(x, off, 64);
            if (lane >= off) x += y;
        }
        x *= RCP_LN2_F;
        const float xl = __shfl(x, 63, 64);      // rows past the end carry the last valid sum
        const float ex = fast_exp2(x);
        sGB[(2 * m) * CH + lane] = x;
        sGB[(2 * m + 1) * CH + lane] = b;
        float* tab = (float*)(p.ws.Rec + (ci * HV + hv) * REC_BYTES + REC_TAB);
        const float nk = sRN[lane], nq = sRN[CH + lane];
        tab[TAB_DEC + lane] = fast_exp2(xl - x) * nk;        // multiplies v_new rows on their way into k^T v_new
        tab[TAB_SG + lane] = p.scale * ex * nq;              // multiplies (q S) rows
        tab[TAB_EG + lane] = ex * nk;                        // multiplies (k S) rows
        if (lane == 63) tab[TAB_GLAST] = x;
        float* tab2 = (float*)(p.ws.Rec + (ci * HV + hv) * REC_BYTES + REC_TAB2);
        tab2[TAB2_G + lane] = x;
        tab2[TAB2_NQS + lane] = p.scale * nq;
        tab2[TAB2_NK + lane] = nk;
    }

    // |k_t|^2 is the diagonal of K K^T: lane (c16, g) of the diagonal tile holds rows 4g .. 4g+3 of column c16
    {
        float d = 0.f;
#pragma unroll
        for (int tj = 0; tj < 4; ++tj)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (tj == w && r == (c16 & 3)) d = kk[tj][r];
        if ((c16 >> 2) == g) sRN[2 * CH + 16 * w + c16] = d;
    }
    __syncthreads();     // k and q are dead from here on: their bytes become L and X
    // ---- bound on the chunk's transition, per value head: every token contributes gamma_t max(1, |1 - beta_t |k~_t|^2|)
    // (rows past the end have beta = 0 and g = 0) ----
    for (int m = w; m < G; m += 4) {
        const float nk = sRN[lane];
        float lb = fabsf(1.f - sGB[(2 * m + 1) * CH + lane] * sRN[2 * CH + lane] * nk * nk);
        lb = lb > 1.f ? __log2f(lb) : 0.f;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) lb += __shfl_xor(lb, off, 64);
        if (lane == 63) p.ws.Bound[ci * HV + h * G + m] = sGB[(2 * m) * CH + 63] + lb;
    }
    // P of every value head first: the raw q K^T tiles then leave the registers before the inversion needs them
    for (int m = 0; want_P && m < G; ++m) {
        const int hv = h * G + m;
        const float* sG = sGB + (2 * m) * CH;
        char* rec = p.ws.Rec + (ci * HV + hv) * REC_BYTES;
        // ---- P^T tiles of query tile tt (gated, lower incl. diagonal), straight to memory ----
        {
            const int t = 16 * tt + c16;
            const float gt = sG[t], st = p.scale * sRN[CH + t];
#pragma unroll
            for (int sp = 0; sp < 2; ++sp) {
                if (tt < 2 && sp == 1) continue;        // identically zero, not stored
                V8 frag;
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int tj = 2 * sp + half;
                    if (tj > tt) {              // a key tile after the query tile: zero (tt is scalar: nothing is evaluated)
#pragma unroll
                        for (int r = 0; r < 4; ++r) frag[half * 4 + r] = from_f32<T>(0.f);
                        continue;
                    }
                    const f32x4 gj = *(const f32x4*)(sG + 16 * tj + 4 * g), nj = *(const f32x4*)(sRN + 16 * tj + 4 * g);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int j = 16 * tj + 4 * g + r;
                        const float val = (t >= j) ? st * nj[r] * qk[tj][r] * fast_exp2(gt - gj[r]) : 0.f;
                        frag[half * 4 + r] = from_f32<T>(val);
                    }
                }
                store_frag<T>(rec + REC_P, tt, sp, lane, frag);
            }
        }
    }
    for (int m = 0; m < G; ++m) {
        const int hv = h * G + m;
        const float* sG = sGB + (2 * m) * CH;
        const float* sB = sG + CH;
        char* rec = p.ws.Rec + (ci * HV + hv) * REC_BYTES;
        // ---- L tiles of row-tile w (gated, beta-scaled, strictly lower) ----
        {
            const f32x4 gi = *(const f32x4*)(sG + 16 * w + 4 * g);
            const f32x4 bi = *(const f32x4*)(sB + 16 * w + 4 * g) * *(const f32x4*)(sRN + 16 * w + 4 * g);
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                const int j = 16 * tj + c16;
                if (tj > w) {                   // above the diagonal: zero (w is scalar: nothing is evaluated)
                    if (w < 2 && tj >= 2) {     // only the block that will hold XT is ever read
#pragma unroll
                        for (int r = 0; r < 4; ++r) sL[(16 * w + 4 * g + r) * LP + j] = 0.f;
                    }
                    continue;
                }
                const float gj = sG[j], nj = sRN[j];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    // select, never multiply by a mask: 2^(G_i-G_j) may overflow above the diagonal
                    const float val = (i > j) ? bi[r] * nj * kk[tj][r] * fast_exp2(gi[r] - gj) : 0.f;
                    sL[i * LP + j] = val;
                    if (tj == w) sLd[(w * 16 + c16) * 16 + 4 * g + r] = val;
                }
            }
        }
        __syncthreads();     // L complete

        // ---- X = (I+L)^-1: 16x16 diagonal blocks by forward substitution.  Lane c16 owns column c16 of
        // the block; as soon as x_j is known it is folded into the pending sums of all later rows, so
        // the dependent chain is 16 steps of two operations (not the 120 of a row-by-row evaluation).
        {
            const int b0 = 16 * w;
            const float* ld = sLd + w * 256;
            float x[16], acc[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                x[j] = ((j == c16) ? 1.f : 0.f) - acc[j];
                float col[16];
#pragma unroll
                for (int q4 = (j + 1) / 4; q4 < 4; ++q4) *(f32x4*)(col + 4 * q4) = *(const f32x4*)(ld + j * 16 + 4 * q4);
#pragma unroll
                for (int i = j + 1; i < 16; ++i) acc[i] += col[i] * x[j];
            }
            if (g == 0) {
#pragma unroll
                for (int i = 0; i < 16; ++i) sX[(b0 + i) * LP + b0 + c16] = x[i];
            }
            // The merges below multiply by X blocks from the left AND from the right.  A right factor is read by
            // columns, so it is kept transposed as well (one 16-byte LDS read then serves four matrix
            // instructions): XT, the transposed top-left 32x32 block, lives in the unused upper-right
            // block of L (zero so far), the transposed X22 in rows 16..31 of the unused upper-right block of X.
            if (g == 1) {
                float* xt = (w < 2) ? sL + (b0 + c16) * LP + 32 + b0 : sX + (16 + c16) * LP + 32;
                if (w != 3) {
#pragma unroll
                    for (int i4 = 0; i4 < 4; ++i4) *(f32x4*)(xt + 4 * i4) = f32x4{x[4 * i4], x[4 * i4 + 1], x[4 * i4 + 2], x[4 * i4 + 3]};
                }
            }
            // zero tile above the diagonal inside each 32x32 diagonal block
            if ((w & 1) == 0) {
#pragma unroll
                for (int r = 0; r < 4; ++r) sX[(b0 + 4 * g + r) * LP + b0 + 16 + c16] = 0.f;
            }
        }
        __syncthreads();
        // 16x16 products on the fp32 matrix cores, contraction over 16*nq indices: A by rows (pitch LP),
        // the right factor transposed (Bt[n][k], pitch LP); step e of block q uses the indices {16q + 4g + e}
        auto mm_rt = [&](const float* A, const float* Bt, int nq) {
            f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                if (q >= nq) break;
                const f32x4 a = *(const f32x4*)(A + c16 * LP + 16 * q + 4 * g);
                const f32x4 bt = *(const f32x4*)(Bt + c16 * LP + 16 * q + 4 * g);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[q] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], bt[e], acc[q], 0, 0, 0);
            }
            return acc[0] + acc[1];
        };
        // ---- merge 16 -> 32: X[hi][lo] = -X[hi][hi] (L[hi][lo] X[lo][lo]); pairs (1,0) and (3,2) by waves 0 and 1.
        // A wave only reads back what it has written itself (LDS operations of a wave execute in order), so
        // there is no barrier between the two products; waves 2 and 3 leave their SIMDs to other workgroups.
        if (w < 2) {
            const int hi = 2 * w + 1, lo = 2 * w;
            float* tmpT = sX + 32 + 16 * w;                     // rows 0..15 of the unused upper-right block: (L X)^T
            const float* xlo_t = w ? sX + 16 * LP + 32 : sL + 32;
            const f32x4 y = mm_rt(sL + (16 * hi) * LP + 16 * lo, xlo_t, 1);
            *(f32x4*)(tmpT + c16 * LP + 4 * g) = y;
            const f32x4 z = mm_rt(sX + (16 * hi) * LP + 16 * hi, tmpT, 1);
#pragma unroll
            for (int r = 0; r < 4; ++r) sX[(16 * hi + 4 * g + r) * LP + 16 * lo + c16] = -z[r];
            if (w == 0) *(f32x4*)(sL + c16 * LP + 32 + 16 + 4 * g) = -z;             // X10 into XT
        }
        __syncthreads();
        // ---- merge 32 -> 64: X[32:64][0:32] = -X[32:64][32:64] (L[32:64][0:32] X[0:32][0:32]) ----
        {
            const int a = w >> 1, b = w & 1;
            float* tmp2T = sX + 32;                             // rows 0..31, columns 32..63: (L X)^T
            const f32x4 y = mm_rt(sL + (32 + 16 * a) * LP, sL + (16 * b) * LP + 32, 2);
            *(f32x4*)(tmp2T + (16 * b + c16) * LP + 16 * a + 4 * g) = y;
            __syncthreads();
            const f32x4 z = mm_rt(sX + (32 + 16 * a) * LP + 32, tmp2T + (16 * b) * LP, 2);
#pragma unroll
            for (int r = 0; r < 4; ++r) sX[(32 + 16 * a + 4 * g + r) * LP + 16 * b + c16] = -z[r];
        }
        __syncthreads();
        // ---- Xb = X diag(beta) rows of t-tile w as A-operand fragments ----
        {
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
                store_frag<T>(rec + REC_X, w, sp, lane, frag);
            }
        }
        if (m + 1 < G) __syncthreads();          // the next value head overwrites L and X
    }
}

template <typename T>
int launch_prepare(const ChunkParams& p, int64_t num_chunks, hipStream_t stream) {
    auto kern = gdn_chunk_prepare_kernel<T>;
    const int G = p.HV / p.H;
    const size_t smem = prep_smem(G);
    if (smem > 64 * 1024) {
        set_error("gdn_chunk_fwd: %d value heads per q/k head exceed what the prepare kernel stages", G);
        return GDN_ERR_UNSUPPORTED;
    }
    static SmemAttrDone attr_done;       // per instantiation
    if (int rc = ensure_dynamic_smem((const void*)kern, 64 * 1024, attr_done, "hipFuncSetAttribute(prepare)")) return rc;
    dim3 grid((unsigned)(num_chunks * p.H)), block(256);
    hipLaunchKernelGGL(kern, grid, block, smem, stream, p);
    return check_launch("gdn_chunk_prepare_kernel");
}
template int launch_prepare<bf16_t>(const ChunkParams&, int64_t, hipStream_t);
template int launch_prepare<f16_t>(const ChunkParams&, int64_t, hipStream_t);

}  // namespace gdn
