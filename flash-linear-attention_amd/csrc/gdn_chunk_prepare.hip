// Chunk-parallel stage of the chunked prefill: one WAVE per (chunk, value head) computes what does not depend on the
// running state and is not a plain copy of the inputs:
//   G = cumsum(g)/ln2,  L = beta*(K K^T)*2^(G_i-G_j) (i>j),  X = (I+L)^-1 in fp32,  Xb = X diag(beta),
//   the per-token gate tables, a bound on the chunk's transition, and on request P = scale*tril(q k^T * 2^(G_i-G_j)).
// Optional prologues of the reference are folded in: the gate and beta activations, and the l2 normalisation of k as
// per-row factors 1/|k_t| on L and the tables (so the sequential stage reads q and k exactly as the caller gave them;
// q is read here only for P, its row factors 1/|q_t| are applied by the scan where it has q in LDS anyway).  Xb and P are written in the exact register order ("fragments") in which the scan kernel feeds
// them to the matrix cores; the scan forms v_new = Xb (v - 2^G (k S)) itself from the raw k and v, so neither
// w = Xb 2^G k nor u = Xb v is ever materialised.
//
// A wave shares nothing with the other waves of its workgroup, so there is no workgroup barrier:
//   * The k rows are loaded straight into matrix-core operand registers (the operand layout of A and of B is the same:
//     lane (c16, g) holds 8 features of token row c16), so K K^T needs no LDS; the value heads of a q/k head sit in
//     neighbouring waves and read the same lines.
//   * Everything is kept TRANSPOSED: the raw tile (a, b), a <= b, holds (k_j . k_i) for rows j of t-tile a and columns i
//     of t-tile b, gated it is U = L^T, and T = X^T = (I + U)^-1 is upper triangular.  A tile in accumulator layout
//     (lane (c16, g): rows 4g..4g+3, column c16) serves directly as the RIGHT factor of a product on the fp32 matrix
//     cores (step e contracts over the indices {4g + e}), the left factor comes from LDS by rows, and the result is
//     again in accumulator layout.  The transposed X in accumulator layout is also exactly the order of the Xb operand
//     fragments (row c16, columns 4g + e): results go from registers to memory.
//   * Diagonal 16x16 blocks: lane group g inverts block g by substitution, one row of X per lane (all 64 lanes busy).
//     Merges: T(lo,hi) = -(T(lo,lo) U(lo,hi)) T(hi,hi) on 16-tiles, then on 32-blocks with the zero tiles left out: the gated
//     tiles U are right factors and never leave the registers, only the products T U pass through LDS.
#include "gdn_chunk_common.h"

namespace gdn {

// LDS per wave: seven 16x16 fp32 tiles that serve as left factors.  The diagonal blocks of L (by rows) and the three gate
// tables lie where the transposed diagonal blocks of X go afterwards, |k|^2 and 1/|q| where the first products go
// afterwards: 8.75 KB, four workgroups per CU.
constexpr int TP = 20;                                       // pitch (floats) of a 16x16 fp32 tile in LDS
constexpr int PW_FLOATS = 7 * 16 * TP;                       // 2240 floats per wave
constexpr int PW_WAVES = 4;                                  // waves per workgroup: small workgroups keep the CU's wave slots filled
constexpr size_t PREP_SMEM = (size_t)PW_WAVES * PW_FLOATS * 4;

// WANT_P: also the records' P (for callers that look at the records; the scan kernels form P themselves): keeps the q
// rows in registers beside the k rows, so half as many waves fit.
template <typename T, bool WANT_P>
__global__ __launch_bounds__(64 * PW_WAVES, (WANT_P ? 8 : 16) / PW_WAVES) void gdn_chunk_prepare_kernel(ChunkParams p, int64_t units) {
    typedef typename Mma<T>::V8 V8;
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, c16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t u = (int64_t)blockIdx.x * PW_WAVES + w;    // (chunk, value head), heads fastest
    if (u >= units) return;
    float* base = (float*)smem + w * PW_FLOATS;
    float* tiles = base;
    // left factors: the transposed diagonal blocks T(0,0) .. T(3,3) and the intermediate products V = T U; the gated
    // tiles U themselves stay in registers as right factors
    constexpr int I_T00 = 0, I_T11 = 1, I_T22 = 2, I_T33 = 3, I_V01 = 4, I_V23 = 5, I_T01 = I_V01;
    constexpr int I_V02 = I_T22, I_V03 = I_T33, I_V12 = I_V23, I_V13 = 6;      // (T(2,2), T(3,3), V(2,3) are in registers by then)
    float* sLd = tiles;                                      // [4][16 i][16 j] diagonal blocks of L, by rows (until the T(g,g) are written)
    float* sG = tiles + 1024; float* sBN = sG + 64; float* sNK = sG + 128;      // gate tables (likewise)
    float* sK2 = tiles + 4 * 16 * TP; float* sNQ = sK2 + 64; // (until the gated tiles are written)
    auto tile = [&](int i) { return tiles + i * 16 * TP; };
    auto lds_sync = [] { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };   // (LDS operations of a wave execute in order)

    const int H = p.H, HV = p.HV, G = HV / H, K = p.K;
    const int64_t ci = u / HV;
    const int hv = (int)(u % HV), h = hv / G;
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
    const bool l2 = p.flags & GDN_FLAG_QK_L2NORM;      // k is l2-normalised here, as row factors (q: by the scan, or below for P)
    const bool q_norms_here = l2 && !(p.flags & FLAG_Q_NORM_IN_SCAN);       // 1/|q_t| into the tables (else the scan applies it)

    // ---- loads: the gate inputs of token `lane`, then the k rows as operand fragments ----
    // (as raw bits, converted where they are used: a 16-bit value converted on the spot would hold the k rows' requests back
    // until it has arrived)
    uint32_t rg = 0, rb = 0;
    if (lane < valid) {
        rg = p.g ? load_scalar_bits(p.g, (tok0 + lane) * HV + hv, p.gb_dtype) : 0;   // (no gate: the plain delta rule)
        rb = load_scalar_bits(p.beta, (tok0 + lane) * HV + hv, p.gb_dtype);
    }
    f32x4 U[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = a; b < 4; ++b) U[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    float sq[4] = {0.f, 0.f, 0.f, 0.f};
    f32x4 QK[4][4];                              // (WANT_P) raw k q^T tiles, like U
    if constexpr (WANT_P) {
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = a; b < 4; ++b) QK[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    {
        const T* kg = (const T*)p.k + (tok0 * H + h) * K;
        const T* qg = (const T*)p.q + (tok0 * H + h) * K;
        const u32x4 z = {0u, 0u, 0u, 0u};
        // one 32-bit offset per lane (its row of a t-tile, its 8 features of a 32-feature block); tile and block
        // select a wave-uniform base
        const uint32_t lane_off = ((uint32_t)c16 * (uint32_t)(H * K) + 8u * g) * (uint32_t)sizeof(T);
        // (a full chunk with the 32 features in range - the common case - loads without any per-lane condition)
        auto fragment = [&](const T* rows, int t, int col0) {
            const char* bp = (const char*)(rows + (int64_t)(16 * t) * H * K + col0);
            if (valid == CH && col0 + 32 <= K) return *(const u32x4*)(bp + lane_off);
            return (16 * t + c16 < valid && col0 + 8 * g < K) ? *(const u32x4*)(bp + lane_off) : z;
        };
        // 128 features at a time: all 16 fragments of a round are requested before the first product; the q rows (for
        // their norms only) follow into the same registers once the products have been issued
        for (int k0 = 0; k0 < K; k0 += 128) {
            u32x4 fk[4][4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) fk[t][s4] = fragment(kg, t, k0 + 32 * s4);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = a; b < 4; ++b)
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4)
                        U[a][b] = Mma<T>::run(__builtin_bit_cast(V8, fk[a][s4]), __builtin_bit_cast(V8, fk[b][s4]), U[a][b]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (WANT_P) {
                u32x4 fq[4][4];
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4) fq[t][s4] = fragment(qg, t, k0 + 32 * s4);
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int b = a; b < 4; ++b)
#pragma unroll
                        for (int s4 = 0; s4 < 4; ++s4)      // rows: key tokens of tile a, column: query token 16b + c16
                            QK[a][b] = Mma<T>::run(__builtin_bit_cast(V8, fk[a][s4]), __builtin_bit_cast(V8, fq[b][s4]), QK[a][b]);
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4) {
                        const V8 q8 = __builtin_bit_cast(V8, fq[t][s4]);
#pragma unroll
                        for (int e = 0; e < 8; ++e) { const float x = to_f32(q8[e]); sq[t] += x * x; }
                    }
            } else if (q_norms_here) {                       // the q rows into the registers that held k
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4) fk[t][s4] = fragment(qg, t, k0 + 32 * s4);
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4) {
                        const V8 q8 = __builtin_bit_cast(V8, fk[t][s4]);
#pragma unroll
                        for (int e = 0; e < 8; ++e) { const float x = to_f32(q8[e]); sq[t] += x * x; }
                    }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    // |k_t|^2 is the diagonal of K K^T; |q_t|^2 (for P only) is summed over the four lanes that share a row
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        float d = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (r == (c16 & 3)) d = U[t][t][r];
        if ((c16 >> 2) == g) sK2[16 * t + c16] = d;
        if (WANT_P || q_norms_here) {
            float a = sq[t];
            a += __shfl_xor(a, 16, 64);
            a += __shfl_xor(a, 32, 64);
            if (g == t) sNQ[16 * t + c16] = l2 ? rsqrtf(a + 1e-6f) : 1.f;
        }
    }
    lds_sync();
    // ---- gates: inclusive scan over the chunk, one token per lane; the tables; the bound on the chunk's transition ----
    float beta_tok;
    {
        float x = scalar_of_bits(rg, p.gb_dtype), b = scalar_of_bits(rb, p.gb_dtype);
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
        const float k2 = sK2[lane];
        const float nk = l2 ? rsqrtf(k2 + 1e-6f) : 1.f, nq = q_norms_here ? sNQ[lane] : 1.f;
        beta_tok = b;
        sG[lane] = x;
        sBN[lane] = b * nk;
        sNK[lane] = nk;
        float* tab = (float*)(p.ws.Rec + (ci * HV + hv) * REC_BYTES + REC_TAB);
        tab[TAB_DEC + lane] = fast_exp2(xl - x) * nk;        // multiplies v_new rows on their way into k^T v_new
        tab[TAB_SG + lane] = p.scale * ex * nq;              // multiplies (q S) rows (nq = 1: the scan adds 1/|q_t|)
        tab[TAB_EG + lane] = ex * nk;                        // multiplies (k S) rows
        if (lane == 63) tab[TAB_GLAST] = x;
        float* tab2 = (float*)(p.ws.Rec + (ci * HV + hv) * REC_BYTES + REC_TAB2);
        tab2[TAB2_G + lane] = x;
        tab2[TAB2_NQS + lane] = p.scale * nq;
        tab2[TAB2_NK + lane] = nk;
        // every token contributes gamma_t max(1, |1 - beta_t |k~_t|^2|) (rows past the end have beta = 0 and g = 0)
        float lb = fabsf(1.f - b * k2 * nk * nk);
        lb = lb > 1.f ? __log2f(lb) : 0.f;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) lb += __shfl_xor(lb, off, 64);
        if (lane == 63) p.ws.Bound[ci * HV + hv] = x + lb;
    }
    lds_sync();
    if constexpr (WANT_P) {
        // ---- P^T tiles (rows: key tokens j, column: query token t; lower triangle incl. the diagonal), gated, as fragments ----
        char* rec = p.ws.Rec + (ci * HV + hv) * REC_BYTES;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const float gt = sG[16 * b + c16], st = p.scale * sNQ[16 * b + c16];
#pragma unroll
            for (int sp = 0; sp < 2; ++sp) {
                if (b < 2 && sp == 1) continue;         // identically zero, not stored
                V8 frag;
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int a = 2 * sp + half;
                    if (a > b) {                        // a key tile after the query tile: zero
#pragma unroll
                        for (int r = 0; r < 4; ++r) frag[half * 4 + r] = from_f32<T>(0.f);
                        continue;
                    }
                    const f32x4 gj = *(const f32x4*)(sG + 16 * a + 4 * g), nj = *(const f32x4*)(sNK + 16 * a + 4 * g);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const bool below = a < b || c16 >= 4 * g + r;
                        frag[half * 4 + r] = from_f32<T>(below ? st * nj[r] * QK[a][b][r] * fast_exp2(gt - gj[r]) : 0.f);
                    }
                }
                store_frag<T>(rec + REC_P, b, sp, lane, frag);
            }
        }
    }
    // ---- U = L^T: gated, beta-scaled, strictly upper; diagonal blocks to LDS as L by rows, the others as left factors ----
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = a; b < 4; ++b) {
            const float gi = sG[16 * b + c16], bni = sBN[16 * b + c16];               // column: token i
            const f32x4 gj = *(const f32x4*)(sG + 16 * a + 4 * g), nj = *(const f32x4*)(sNK + 16 * a + 4 * g);   // rows: tokens j
            f32x4 val;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // select, never multiply by a mask: 2^(G_i-G_j) may overflow for i < j
                const bool below = a < b || c16 > 4 * g + r;
                val[r] = below ? bni * nj[r] * U[a][b][r] * fast_exp2(gi - gj[r]) : 0.f;
            }
            if (a == b) *(f32x4*)(sLd + a * 256 + c16 * 16 + 4 * g) = val;             // L[i = c16][j = 4g + r]
            else U[a][b] = val;                                                        // stays in registers: a right factor
        }
    lds_sync();
    // ---- diagonal blocks: X (I + L) = I by rows, from the right.  Lane c16 of group g owns row c16 of block g; as soon as
    // x_i is known it is folded into the pending sums of all earlier columns (a dependent chain of 16 short steps) ----
    {
        const float* ld = sLd + g * 256;
        float x[16], acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int i = 15; i >= 0; --i) {
            x[i] = ((i == c16) ? 1.f : 0.f) - acc[i];
            float row[16];
#pragma unroll
            for (int q4 = 0; q4 < (i + 3) / 4; ++q4) *(f32x4*)(row + 4 * q4) = *(const f32x4*)(ld + i * 16 + 4 * q4);
#pragma unroll
            for (int j = 0; j < i; ++j) acc[j] += row[j] * x[i];
        }
        // T(g,g) = X_gg^T as a left factor: [row j][column c16]
        float* tt = tile(I_T00 + g);             // (group g: block g)
#pragma unroll
        for (int j = 0; j < 16; ++j) tt[j * TP + c16] = x[j];
    }
    lds_sync();
    auto acc_layout = [&](int i) {               // a tile of LDS in accumulator layout
        const float* t = tile(i);
        return f32x4{t[(4 * g) * TP + c16], t[(4 * g + 1) * TP + c16], t[(4 * g + 2) * TP + c16], t[(4 * g + 3) * TP + c16]};
    };
    // acc + A B: A a tile of LDS by rows, B in accumulator layout
    auto mul = [&](int ia, f32x4 B, f32x4 acc) {
        const f32x4 a = *(const f32x4*)(tile(ia) + c16 * TP + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], B[e], acc, 0, 0, 0);
        return acc;
    };
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    auto put = [&](int i, f32x4 v) {             // a tile in accumulator layout to LDS, by rows
#pragma unroll
        for (int r = 0; r < 4; ++r) tile(i)[(4 * g + r) * TP + c16] = v[r];
    };
    const f32x4 T00 = acc_layout(I_T00), T11 = acc_layout(I_T11), T22 = acc_layout(I_T22), T33 = acc_layout(I_T33);
    // ---- merge 16 -> 32: T(lo,hi) = -(T(lo,lo) U(lo,hi)) T(hi,hi) ----
    put(I_V01, mul(I_T00, U[0][1], zero));
    put(I_V23, mul(I_T22, U[2][3], zero));
    lds_sync();
    const f32x4 T01 = -mul(I_V01, T11, zero);
    const f32x4 T23 = -mul(I_V23, T33, zero);
    put(I_T01, T01);
    lds_sync();
    // ---- merge 32 -> 64: V = T[0:32][0:32] U[0:32][32:64], T[0:32][32:64] = -V T[32:64][32:64] (zero tiles left out) ----
    put(I_V02, mul(I_T00, U[0][2], mul(I_T01, U[1][2], zero)));
    put(I_V03, mul(I_T00, U[0][3], mul(I_T01, U[1][3], zero)));
    put(I_V12, mul(I_T11, U[1][2], zero));
    put(I_V13, mul(I_T11, U[1][3], zero));
    lds_sync();
    const f32x4 T02 = -mul(I_V02, T22, zero), T03 = -mul(I_V03, T33, mul(I_V02, T23, zero));
    const f32x4 T12 = -mul(I_V12, T22, zero), T13 = -mul(I_V13, T33, mul(I_V12, T23, zero));
    // ---- Xb = X diag(beta) as operand fragments: rows of t-tile tt, columns {32sp + 4g + e} and {32sp + 16 + 4g + e} ----
    {
        char* rec = p.ws.Rec + (ci * HV + hv) * REC_BYTES;
        auto emit = [&](int tt, int sp, f32x4 lo, f32x4 hi, bool has_hi) {
            V8 frag;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                frag[e] = from_f32<T>(lo[e] * __shfl(beta_tok, 32 * sp + 4 * g + e, 64));
                frag[4 + e] = from_f32<T>(has_hi ? hi[e] * __shfl(beta_tok, 32 * sp + 16 + 4 * g + e, 64) : 0.f);
            }
            store_frag<T>(rec + REC_X, tt, sp, lane, frag);
        };
        emit(0, 0, T00, zero, false);
        emit(1, 0, T01, T11, true);
        emit(2, 0, T02, T12, true);
        emit(2, 1, T22, zero, false);
        emit(3, 0, T03, T13, true);
        emit(3, 1, T23, T33, true);
    }
}

template <typename T, bool WANT_P>
static int launch_prepare_as(const ChunkParams& p, int64_t units, hipStream_t stream) {
    auto kern = gdn_chunk_prepare_kernel<T, WANT_P>;
    static SmemAttrDone attr_done;       // per instantiation
    if (int rc = ensure_dynamic_smem((const void*)kern, PREP_SMEM, attr_done, "hipFuncSetAttribute(prepare)")) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)((units + PW_WAVES - 1) / PW_WAVES)), dim3(64 * PW_WAVES), PREP_SMEM, stream, p, units);
    return check_launch("gdn_chunk_prepare_kernel");
}

template <typename T>
int launch_prepare(const ChunkParams& p, int64_t num_chunks, hipStream_t stream) {
    const int64_t units = num_chunks * p.HV;
    if (units <= 0) return GDN_OK;
    return p.want_P ? launch_prepare_as<T, true>(p, units, stream) : launch_prepare_as<T, false>(p, units, stream);
}
template int launch_prepare<bf16_t>(const ChunkParams&, int64_t, hipStream_t);
template int launch_prepare<f16_t>(const ChunkParams&, int64_t, hipStream_t);

}  // namespace gdn
