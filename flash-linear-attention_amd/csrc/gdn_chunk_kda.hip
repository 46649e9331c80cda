// Chunked forward of the KDA operator (the gated delta rule with a decay per key feature), 64-token chunks, K, V <= 128
// (zero-padded to 128 by the host).  Replaces chunk_kda_fwd (fla/ops/kda/chunk_fwd.py:20-134): the gate activation and
// chunk-local cumsum (fla/ops/kda/gate.py), the intra-chunk stage (fla/ops/kda/chunk_intra.py), recompute_w_u_fwd
// (fla/ops/kda/wy_fast.py), chunk_gated_delta_rule_fwd_h and chunk_gla_fwd_o_gk.  Two kernels:
//
//   prepare  per (chunk, v-head): Gam = cumsum of the log decays inside the chunk [64][K];
//            M_ij = sum_k k_ik k_jk e^(Gam_ik - Gam_jk) (i > j),  P_ij = scale sum_k q_ik k_jk e^(Gam_ik - Gam_jk) (i >= j);
//            A = (I + diag(beta) M)^-1,  w = A (beta k e^Gam),  u = A (beta v);
//            also qg = scale q e^Gam, kg = k e^(Gam_last - Gam), e^Gam_last: what the scan needs, so that it never sees a gate
//   scan     per (sequence, v-head, VBT value columns), chunks in order, state slice in registers:
//            v_new = u - w S;  o = qg S + P v_new;  S <- diag(e^Gam_last) S + kg^T v_new
//
// The exponent Gam_ik - Gam_jk is only ever non-positive for i >= j, but it cannot be split into a factor of row i and a
// factor of row j without overflow unless a reference row lies between them.  Blocks of 16 rows: for j in an earlier
// block than i the reference is the last row in front of i's block, e^(Gam_i - ref) e^(ref - Gam_j) with both exponents <= 0,
// and the products run on the matrix cores; inside a 16 x 16 diagonal block every pair gets its own exponentials
// (the reference does the same, fla/ops/kda/chunk_intra.py: sub-chunks of 16).
//
// The comba operator (one decay per token and head, a second key p for the prediction, which sees the state before the
// token's decay; fla/ops/comba/chunk.py:22-90) has a prepare kernel of its own that writes the same per-chunk operands,
// and shares the scan:  M_ij = (p_i . k_j) e^(Gam0_i - Gam_j) with Gam0 = Gam - g,  w = A (beta p e^Gam0).
#include "gdn_chunk_kda.h"

namespace gdn {

// ---------------------------------------------------------------------------------------------
// prepare
// ---------------------------------------------------------------------------------------------
// Two workgroups share a CU (80 KB of LDS each; a workgroup's phases are chains of dependent steps - the substitution above all -
// that leave most of a CU idle): only k is kept as a tile; a wave reads nothing of q but its own 16 rows, which stay in
// registers as operand fragments from the load to the store of qg; v arrives late, in the place of the matrix L.
static_assert(64 * PL * 4 == 64 * P128 * 2, "the rows of v take the place of the matrix L");
constexpr size_t KDA_PREP_SMEM = (2 * 64 * P128 + 64 * P64) * 2 + (64 * PG + 64) * 4;

template <typename T>
__global__ __launch_bounds__(256, 2) void gdn_kda_prepare_kernel(KdaParams p, int64_t units) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    T* sK = (T*)smem; T* sV = sK + 64 * P128; T* sA = sV + 64 * P128;
    float* sL = (float*)sV;
    float* sG = (float*)(sA + 64 * P64); float* sBeta = sG + 64 * PG;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;

    // A workgroup walks over the units; the next unit's rows and gates are fetched into registers meanwhile.
    TileRegs<BD> rK, rV;
    V8 rQ[4];                                                   // q: row 16w + c16, features 32s + 8g .. + 7
    float rG[32];                                               // gates: a thread per key feature and half of the chunk's rows
    uint32_t rB = 0;                                            // (raw bits: converted when the unit's turn comes)
    // (the lane number is an argument: inside the loop over the units it is the opaque copy, see there)
    auto fetch_v = [&](int64_t u, int tid) {
        const ChunkAt c = chunk_at(p, u / p.HV);
        fetch_tile<BD>(rV, (const T*)p.v + (c.tok0 * p.HV + (int)(u % p.HV)) * BD, (int64_t)p.HV * BD, c.valid, tid);
    };
    auto fetch = [&](int64_t u, int tid) {
        const int lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
        const int hv = (int)(u % p.HV), hq = hv / (p.HV / p.H);
        const ChunkAt c = chunk_at(p, u / p.HV);
        fetch_tile<BD>(rK, (const T*)p.k + (c.tok0 * p.H + hq) * BD, (int64_t)p.H * BD, c.valid, tid);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
#pragma unroll
            for (int e = 0; e < 8; ++e) rQ[s][e] = (T)0.f;
            if (16 * w + c16 < c.valid) rQ[s] = *(const V8*)((const T*)p.q + ((c.tok0 + 16 * w + c16) * p.H + hq) * BD + 32 * s + 8 * g);
        }
        rB = (tid < 64 && tid < c.valid) ? load_scalar_bits(p.beta, (c.tok0 + tid) * p.HV + hv, p.gb_dtype) : 0;
    };
    auto fetch_g = [&](int64_t u, int tid) {
        const int hv = (int)(u % p.HV);
        const ChunkAt c = chunk_at(p, u / p.HV);
        const int col = tid & 127, half = tid >> 7;
#pragma unroll
        for (int r = 0; r < 32; ++r) {
            const int row = 32 * half + r;
            rG[r] = row < c.valid ? p.g[((c.tok0 + row) * p.HV + hv) * BD + col] : 0.f;
        }
    };
    fetch(blockIdx.x, tid);
    const int tid_outer = tid;
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
    // (everything derived from the lane number is derived again per unit from a copy the compiler cannot see through: hoisted out
    // of this loop, the addresses of its fully unrolled body would fill the register file before the loop starts, and spill)
    int tid_opaque = tid_outer;
    asm volatile("" : "+v"(tid_opaque));
    const int tid = tid_opaque, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
    const int hv = (int)(u % p.HV);
    const ChunkAt c = chunk_at(p, u / p.HV);
    fetch_g(u, tid);                                                 // (the gates are not fetched ahead: no 32 registers to carry them round the loop)
    put_tile<BD>(sK, P128, rK, tid);
    V8 qx[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) qx[s] = rQ[s];
    {
        // running sums of the gates inside each half of the rows first
        const int col = tid & 127, half = tid >> 7;
        const float a_k = p.gk_act ? (p.A_log ? __expf(p.A_log[hv]) : (p.gk_act == 2 ? 1.f : __expf(1.f))) : 0.f;
        const float bias = (p.gk_act && p.gk_bias) ? p.gk_bias[hv * BD + col] : 0.f;
        float run = 0.f;
#pragma unroll
        for (int r = 0; r < 32; ++r) {
            const int row = 32 * half + r;
            float gt = rG[r];
            if (p.gk_act && row < c.valid) {
                gt += bias;
                gt = p.gk_act == 2 ? p.gk_lower * sigmoid_f(a_k * gt) : -a_k * softplus_f(gt);
            }
            run += gt;
            sG[row * PG + col] = run;
            __builtin_amdgcn_sched_barrier(0);                  // (one row at a time: 32 activations in flight at once cost 100 registers)
        }
    }
    if (tid < 64) {
        float b = scalar_of_bits(rB, p.gb_dtype);
        if ((p.flags & GDN_FLAG_BETA_SIGMOID) && tid < c.valid) b = sigmoid_f(b) * ((p.flags & GDN_FLAG_NEG_EIGVAL) ? 2.f : 1.f);
        sBeta[tid] = b;
    }
    lds_barrier();
    fetch_v(u, tid);
    {
        // second half of the rows: add the first half's total
        const int col = tid & 127, half = tid >> 7;
        if (half == 1) {
            const float tot = sG[31 * PG + col];
#pragma unroll
            for (int r = 0; r < 32; ++r) sG[(32 + r) * PG + col] += tot;
        }
    }
    if (p.flags & GDN_FLAG_QK_L2NORM) {
        // rows of q and k divided by sqrt(sum x^2 + 1e-6).  k: 16 consecutive lanes hold the 16 pieces of a row
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = (tid >> 4) + 16 * i, pc = tid & 15;
            T* at = sK + row * P128 + pc * 8;
            V8 x = *(V8*)at;
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += (float)x[e] * (float)x[e];
            const float r = rsqrtf(sum_over_c16(ss) + 1e-6f);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * r);
            *(V8*)at = x;
        }
        // q: the four lanes that share c16 hold a row
        float ss = 0.f;
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += (float)qx[s][e] * (float)qx[s][e];
        const float r = rsqrtf(sum_over_g(ss) + 1e-6f);
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) qx[s][e] = (T)((float)qx[s][e] * r);
    }
    lds_barrier();

    // ---- M (as L = diag(beta) M, for the substitution) and P, this wave's 16 rows ----
    {
        T* Pu = (T*)p.ws.Pm + u * 64 * 64;
        const int i = 16 * w + c16;                             // the row this lane's operand fragments belong to
        // rows of this block against rows of earlier blocks: reference = the row in front of the block (zeros for block 0)
        V8 kd[4], qd[4];
        const float* gref = sG + (16 * w - 1) * PG + 8 * g;         // the reference row, read where it is used (w > 0)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const float* gi = sG + i * PG + 32 * s + 8 * g;
            const float* gr = sG + (16 * w - 1) * PG + 32 * s + 8 * g;
            const V8 kx = frag_rows(sK, P128, 16 * w, 32 * s, lane);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float f = __expf(gi[e] - (w > 0 ? gr[e] : 0.f));
                kd[s][e] = (T)((float)kx[e] * f);
                qd[s][e] = (T)((float)qx[s][e] * f);
            }
        }
#pragma unroll
        for (int tj = 0; tj < 3; ++tj) {
            if (tj >= w) break;
            f32x4 m = ZERO4, pt = ZERO4;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const float* gj = sG + (16 * tj + c16) * PG + 32 * s + 8 * g;
                V8 kn = frag_rows(sK, P128, 16 * tj, 32 * s, lane);
#pragma unroll
                for (int e = 0; e < 8; ++e) kn[e] = (T)((float)kn[e] * __expf(gref[32 * s + e] - gj[e]));        // (tj < w: w > 0)
                m = Mma<T>::run(kd[s], kn, m);                 // lane: column j = 16tj + c16, rows i = 16w + 4g + r
                pt = Mma<T>::run(kn, qd[s], pt);               // lane: column i = 16w + c16, rows j = 16tj + 4g + r
            }
            const int j = 16 * tj + c16;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int ir = 16 * w + 4 * g + r;
                sL[ir * PL + (j & 3) * 16 + (j >> 2)] = sBeta[ir] * m[r];
            }
            *(V4*)(Pu + i * 64 + 16 * tj + 4 * g) = pack4<T>(pt * p.scale);
        }
        // blocks to the right of the diagonal: zeros
#pragma unroll
        for (int tj = 1; tj < 4; ++tj)
            if (tj > w) *(V4*)(Pu + i * 64 + 16 * tj + 4 * g) = pack4<T>(ZERO4);
        // The diagonal block.  Where the decay across the block stays within what the operand type can hold as a factor
        // e^(ref - Gam_j) >= 1 (the usual case), the same reference serves and the block is one more tile on the matrix
        // cores; otherwise every pair of rows gets its own exponentials.
        float span = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int col = lane + 64 * h;
            span = fminf(span, sG[(16 * w + 15) * PG + col] - (w > 0 ? sG[(16 * w - 1) * PG + col] : 0.f));
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) span = fminf(span, __shfl_xor(span, off, 64));
        constexpr float SPAN_OK = std::is_same<T, bf16_t>::value ? -80.f : -8.f;
        if (span >= SPAN_OK) {
            f32x4 m = ZERO4, pt = ZERO4;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const float* gj = sG + i * PG + 32 * s + 8 * g;
                V8 kn = frag_rows(sK, P128, 16 * w, 32 * s, lane);
#pragma unroll
                for (int e = 0; e < 8; ++e) kn[e] = (T)((float)kn[e] * __expf((w > 0 ? gref[32 * s + e] : 0.f) - gj[e]));
                m = Mma<T>::run(kd[s], kn, m);                 // lane: column j = 16w + c16, rows i = 16w + 4g + r
                pt = Mma<T>::run(kn, qd[s], pt);               // lane: column i = 16w + c16, rows j = 16w + 4g + r
            }
            const int j = 16 * w + c16;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int ir = 16 * w + 4 * g + r;
                sL[ir * PL + (j & 3) * 16 + (j >> 2)] = ir > j ? sBeta[ir] * m[r] : 0.f;
                pt[r] = (16 * w + 4 * g + r) <= i ? pt[r] * p.scale : 0.f;
            }
            *(V4*)(Pu + i * 64 + 16 * w + 4 * g) = pack4<T>(pt);
        } else
        // (lane (c16, g) takes row i against every row j of the block over the features of its own fragments; the four lanes that
        // share a row add up)
        {
#pragma unroll 1
            for (int jl = 0; jl < 16; ++jl) {
                const int rj = 16 * w + jl;
                float mj = 0.f, pj = 0.f;
                if (jl <= c16) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const V8 ki = frag_rows(sK, P128, 16 * w, 32 * s, lane), kj = *(const V8*)(sK + rj * P128 + 32 * s + 8 * g);
                        const float* gi = sG + i * PG + 32 * s + 8 * g;
                        const float* gj = sG + rj * PG + 32 * s + 8 * g;
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const float kk = (float)kj[e] * __expf(gi[e] - gj[e]);
                            mj += (float)ki[e] * kk;
                            pj += (float)qx[s][e] * kk;
                        }
                    }
                }
                mj = sum_over_g(mj); pj = sum_over_g(pj);
                if (g == 0) {
                    sL[i * PL + (rj & 3) * 16 + (rj >> 2)] = jl < c16 ? sBeta[i] * mj : 0.f;
                    Pu[i * 64 + rj] = (T)(jl <= c16 ? p.scale * pj : 0.f);
                }
            }
        }
    }
    lds_barrier();
    solve_unit_lower_blocks<T>(sL, (float*)sA, sA, w, lane);
    lds_barrier();
    if (p.ws.Am) {                                              // (for the backward pass)
        T* Au = (T*)p.ws.Am + u * 64 * 64;
        float* Gu = p.ws.Gk + u * 64 * BD;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = tid + 256 * i, row = idx >> 3, pc = idx & 7;
            *(u32x4*)(Au + row * 64 + pc * 8) = *(const u32x4*)(sA + row * P64 + pc * 8);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int idx = tid + 256 * i, row = idx >> 5, pc = idx & 31;
            *(f32x4*)(Gu + row * BD + pc * 4) = *(const f32x4*)(sG + row * PG + pc * 4);
        }
    }
    {
        // what the scan needs of q and k, and k, v as the factors of w, u
        T* QGu = (T*)p.ws.QG + u * 64 * BD;
        T* KGu = (T*)p.ws.KG + u * 64 * BD;
#pragma unroll
        for (int it = 0; it < 4; ++it) {                        // (the pieces of v: those this thread fetched)
            const int idx = tid + 256 * it, row = idx >> 4, pc = idx & 15;
            const float* gi = sG + row * PG + pc * 8;
            const float* gl = sG + 63 * PG + pc * 8;
            V8 kx = *(V8*)(sK + row * P128 + pc * 8), vx = __builtin_bit_cast(V8, rV.x[it]);
            V8 kg;
            const float b = sBeta[row];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float eg = __expf(gi[e]);
                kg[e] = (T)((float)kx[e] * __expf(gl[e] - gi[e]));
                kx[e] = (T)((float)kx[e] * (b * eg));
                vx[e] = (T)((float)vx[e] * b);
            }
            *(V8*)(KGu + row * BD + pc * 8) = kg;
            *(V8*)(sK + row * P128 + pc * 8) = kx;
            *(V8*)(sV + row * P128 + pc * 8) = vx;                                  // (in the place of L: the substitution is over)
        }
        {
            const int i = 16 * w + c16;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const float* gi = sG + i * PG + 32 * s + 8 * g;
                V8 qg;
#pragma unroll
                for (int e = 0; e < 8; ++e) qg[e] = (T)((float)qx[s][e] * (p.scale * __expf(gi[e])));
                *(V8*)(QGu + i * BD + 32 * s + 8 * g) = qg;
            }
        }
        if (tid < BD) p.ws.EGL[u * BD + tid] = __expf(sG[63 * PG + tid]);
    }
    lds_barrier();
    {
        // w^T and u^T tiles: features on the rows, this wave's 16 tokens on the columns
        T* Wu = (T*)p.ws.Wm + u * 64 * BD;
        T* Uu = (T*)p.ws.Um + u * 64 * BD;
        const int i = 16 * w + c16;
        V8 fa[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) fa[s] = frag_rows(sA, P64, 16 * w, 32 * s, lane);
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            f32x4 aw = ZERO4, au = ZERO4;
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                if (2 * s > w) continue;                        // A is lower triangular
                aw = Mma<T>::run(frag_cols(sK, P128, 32 * s, 16 * n, lane), fa[s], aw);
                au = Mma<T>::run(frag_cols(sV, P128, 32 * s, 16 * n, lane), fa[s], au);
            }
            *(V4*)(Wu + i * BD + 16 * n + 4 * g) = pack4<T>(aw);
            *(V4*)(Uu + i * BD + 16 * n + 4 * g) = pack4<T>(au);
        }
    }
    // (the next unit's rows: requested this late because the phases above have no registers to spare under the cap that lets two
    // workgroups share a CU; the other workgroup covers the wait)
    if (u + gridDim.x < units) fetch(u + gridDim.x, tid);
    lds_barrier();
    }
}

// ---------------------------------------------------------------------------------------------
// prepare, comba
// ---------------------------------------------------------------------------------------------
constexpr size_t COMBA_PREP_SMEM = (4 * 64 * P128 + 64 * P64) * 2 + 3 * 64 * 4;
static_assert(64 * PL * 4 <= 64 * P128 * 2, "the matrix L takes the place of the q tile");

template <typename T>
__global__ __launch_bounds__(256, 2) void gdn_comba_prepare_kernel(KdaParams p, int64_t units) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    T* sK = (T*)smem; T* sQ = sK + 64 * P128; T* sP = sQ + 64 * P128; T* sV = sP + 64 * P128; T* sA = sV + 64 * P128;
    float* sGam = (float*)(sA + 64 * P64); float* sGam0 = sGam + 64; float* sBeta = sGam0 + 64;
    float* sL = (float*)sQ;                                     // once q has been used
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;

    // Two workgroups per CU walk over the units; the next unit's rows and gates are fetched into registers meanwhile.
    TileRegs<BD> rK, rQ, rP, rV;
    uint32_t rG = 0, rB = 0;                                    // (raw bits: converted when the unit's turn comes)
    auto fetch_v = [&](int64_t u) {                             // (on its own, later than the rest: fewer registers live across the substitution)
        const int hv = (int)(u % p.HV);
        const ChunkAt c = chunk_at(p, u / p.HV);
        fetch_tile<BD>(rV, (const T*)p.v + (c.tok0 * p.HV + hv) * BD, (int64_t)p.HV * BD, c.valid, tid);
    };
    auto fetch = [&](int64_t u) {
        const int hv = (int)(u % p.HV), hq = hv / (p.HV / p.H);
        const ChunkAt c = chunk_at(p, u / p.HV);
        fetch_tile<BD>(rK, (const T*)p.k + (c.tok0 * p.H + hq) * BD, (int64_t)p.H * BD, c.valid, tid);
        fetch_tile<BD>(rQ, (const T*)p.q + (c.tok0 * p.H + hq) * BD, (int64_t)p.H * BD, c.valid, tid);
        fetch_tile<BD>(rP, (const T*)p.pk + (c.tok0 * p.H + hq) * BD, (int64_t)p.H * BD, c.valid, tid);
        const bool have = tid < 64 && tid < c.valid;
        rG = have ? load_scalar_bits(p.gs, (c.tok0 + tid) * p.HV + hv, p.gb_dtype) : 0;
        rB = have ? load_scalar_bits(p.beta, (c.tok0 + tid) * p.HV + hv, p.gb_dtype) : 0;
    };
    fetch(blockIdx.x);
    fetch_v(blockIdx.x);
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
    // (everything derived from the lane number is derived again per unit from a copy the compiler cannot see through: hoisted
    // out of this loop, the addresses of its unrolled body would fill the register file and spill)
    int tid_opaque = threadIdx.x;
    asm volatile("" : "+v"(tid_opaque));
    const int tid = tid_opaque, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
    put_tile<BD>(sK, P128, rK, tid);
    put_tile<BD>(sQ, P128, rQ, tid);
    put_tile<BD>(sP, P128, rP, tid);
    put_tile<BD>(sV, P128, rV, tid);
    if (w == 0) {
        const float g_own = scalar_of_bits(rG, p.gb_dtype);
        float run = g_own;                                      // running sum over the chunk's tokens (rows past the end add 0)
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float t = __shfl_up(run, off, 64);
            if (lane >= off) run += t;
        }
        sGam[lane] = run;
        sGam0[lane] = run - g_own;
        sBeta[lane] = scalar_of_bits(rB, p.gb_dtype);
    }
    lds_barrier();
    if (u + gridDim.x < units) fetch(u + gridDim.x);
    if (p.flags & GDN_FLAG_QK_L2NORM) {
        // rows of q, k and p divided by sqrt(sum x^2 + 1e-6): 16 consecutive lanes hold the 16 pieces of a row
#pragma unroll 2
        for (int i = 0; i < 4; ++i) {
            const int row = (tid >> 4) + 16 * i, pc = tid & 15;
#pragma unroll
            for (int which = 0; which < 3; ++which) {
                T* at = (which == 0 ? sK : which == 1 ? sQ : sP) + row * P128 + pc * 8;
                V8 x = *(V8*)at;
                float ss = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) ss += (float)x[e] * (float)x[e];
                const float r = rsqrtf(sum_over_c16(ss) + 1e-6f);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * r);
                *(V8*)at = x;
            }
        }
        lds_barrier();
    }
    const float gl = sGam[63];
    {
        // P, this wave's 16 rows; and what the scan needs of q and k
        T* Pu = (T*)p.ws.Pm + u * 64 * 64;
        const int i = 16 * w + c16;
        V8 qf[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) qf[s] = frag_rows(sQ, P128, 16 * w, 32 * s, lane);
        const float gam_i = sGam[i];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            if (tj > w) { *(V4*)(Pu + i * 64 + 16 * tj + 4 * g) = pack4<T>(ZERO4); continue; }
            f32x4 pt = ZERO4;
#pragma unroll
            for (int s = 0; s < 4; ++s)
                pt = Mma<T>::run(frag_rows(sK, P128, 16 * tj, 32 * s, lane), qf[s], pt);     // lane: column i = 16w + c16, rows j = 16tj + 4g + r
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int jr = 16 * tj + 4 * g + r;
                pt[r] = jr <= i ? p.scale * pt[r] * __expf(gam_i - sGam[jr]) : 0.f;
            }
            *(V4*)(Pu + i * 64 + 16 * tj + 4 * g) = pack4<T>(pt);
        }
        T* QGu = (T*)p.ws.QG + u * 64 * BD;
        T* KGu = (T*)p.ws.KG + u * 64 * BD;
#pragma unroll 2                                        // (unrolled fully, the kernel spills registers)
        for (int it = 0; it < 4; ++it) {
            const int row = (tid >> 4) + 16 * it, pc = tid & 15;
            V8 kx = *(V8*)(sK + row * P128 + pc * 8), qx = *(V8*)(sQ + row * P128 + pc * 8);
            const float fk = __expf(gl - sGam[row]), fq = p.scale * __expf(sGam[row]);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                kx[e] = (T)((float)kx[e] * fk);
                qx[e] = (T)((float)qx[e] * fq);
            }
            *(V8*)(KGu + row * BD + pc * 8) = kx;
            *(V8*)(QGu + row * BD + pc * 8) = qx;
        }
        if (tid < BD) p.ws.EGL[u * BD + tid] = __expf(gl);
    }
    lds_barrier();                                              // q is done with: L takes its place
    {
        // L = diag(beta) M for the substitution, this wave's 16 rows
        V8 pf[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) pf[s] = frag_rows(sP, P128, 16 * w, 32 * s, lane);
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            if (tj > w) continue;
            f32x4 m = ZERO4;
#pragma unroll
            for (int s = 0; s < 4; ++s)
                m = Mma<T>::run(pf[s], frag_rows(sK, P128, 16 * tj, 32 * s, lane), m);       // lane: column j = 16tj + c16, rows i = 16w + 4g + r
            const int j = 16 * tj + c16;
            const float gam_j = sGam[j];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int ir = 16 * w + 4 * g + r;
                sL[ir * PL + (j & 3) * 16 + (j >> 2)] = ir > j ? sBeta[ir] * m[r] * __expf(sGam0[ir] - gam_j) : 0.f;
            }
        }
    }
    lds_barrier();
    solve_unit_lower_blocks<T>(sL, (float*)sA, sA, w, lane);
    {
        // p, v as the factors of w, u
#pragma unroll 2                                        // (unrolled fully, the kernel spills registers)
        for (int it = 0; it < 4; ++it) {
            const int row = (tid >> 4) + 16 * it, pc = tid & 15;
            V8 px = *(V8*)(sP + row * P128 + pc * 8), vx = *(V8*)(sV + row * P128 + pc * 8);
            const float b = sBeta[row], fp = b * __expf(sGam0[row]);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                px[e] = (T)((float)px[e] * fp);
                vx[e] = (T)((float)vx[e] * b);
            }
            *(V8*)(sP + row * P128 + pc * 8) = px;
            *(V8*)(sV + row * P128 + pc * 8) = vx;
        }
    }
    lds_barrier();
    if (u + gridDim.x < units) fetch_v(u + gridDim.x);
    {
        // w^T and u^T tiles: features on the rows, this wave's 16 tokens on the columns
        T* Wu = (T*)p.ws.Wm + u * 64 * BD;
        T* Uu = (T*)p.ws.Um + u * 64 * BD;
        const int i = 16 * w + c16;
        V8 fa[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) fa[s] = frag_rows(sA, P64, 16 * w, 32 * s, lane);
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            f32x4 aw = ZERO4, au = ZERO4;
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                if (2 * s > w) continue;                        // A is lower triangular
                aw = Mma<T>::run(frag_cols(sP, P128, 32 * s, 16 * n, lane), fa[s], aw);
                au = Mma<T>::run(frag_cols(sV, P128, 32 * s, 16 * n, lane), fa[s], au);
            }
            *(V4*)(Wu + i * BD + 16 * n + 4 * g) = pack4<T>(aw);
            *(V4*)(Uu + i * BD + 16 * n + 4 * g) = pack4<T>(au);
        }
    }
    lds_barrier();
    }
}

// ---------------------------------------------------------------------------------------------
// scan: the state slice [128][VBT] lives in registers as transposed tiles (wave w: key rows 32w .. 32w+31 as two tiles a2,
// lane (c16, g): key 16(2w+a2) + c16, value columns 16b + 4g .. +3); the next chunk's tiles are fetched into registers
// while the current chunk is computed.
// ---------------------------------------------------------------------------------------------
// (u comes in, and o leaves, as whole rows through LDS tiles of their own: the lanes that hold them as matrix-instruction operands
// and results would move 8-byte pieces of 16 rows per instruction)
template <int VBT> constexpr size_t kda_scan_smem() { return (3 * 64 * P128 + 64 * P64 + BD * (VBT + 8) + 3 * 64 * (VBT + 8)) * 2 + (BD + 64) * 4; }

template <typename T, int VBT>
__global__ __launch_bounds__(256) void gdn_kda_scan_kernel(KdaParams p) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    constexpr int PV = VBT + 8, NB = VBT / 16, NVS = BD / VBT;
    extern __shared__ __align__(16) char smem[];
    T* sW = (T*)smem; T* sKG = sW + 64 * P128; T* sQG = sKG + 64 * P128; T* sP = sQG + 64 * P128;
    T* sS = sP + 64 * P64; T* sVn = sS + BD * PV; T* sU = sVn + 64 * PV; T* sO = sU + 64 * PV;
    float* sE = (float*)(sO + 64 * PV);
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    const int64_t run = (int64_t)(blockIdx.x / (8 * NVS)) * 8 + blockIdx.x % 8;       // (slices of one head on one XCD)
    if (run >= p.N * p.HV) return;
    const int vs = (blockIdx.x / 8) % NVS, hv = (int)(run % p.HV);
    const int64_t n = run / p.HV;
    const SeqAt sq = seq_at(p, n);
    const int vcol0 = vs * VBT;

    f32x4 S[2][NB];
#pragma unroll
    for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int kk = 16 * (2 * w + a2) + c16;
            S[a2][b] = p.h0 ? *(const f32x4*)(p.h0 + ((n * p.HV + hv) * BD + kk) * BD + vcol0 + 16 * b + 4 * g) : ZERO4;
        }
    TileRegs<BD> rW, rKG, rQG;
    TileRegs<CH> rP;
    TileRegs<VBT> rU;
    float rE = 0.f;
    auto fetch = [&](int64_t ic) {
        const int64_t u = (sq.cbase + ic) * p.HV + hv;
        fetch_tile<BD>(rW, (const T*)p.ws.Wm + u * 64 * BD, BD, 64, tid);
        fetch_tile<BD>(rKG, (const T*)p.ws.KG + u * 64 * BD, BD, 64, tid);
        fetch_tile<BD>(rQG, (const T*)p.ws.QG + u * 64 * BD, BD, 64, tid);
        fetch_tile<CH>(rP, (const T*)p.ws.Pm + u * 64 * 64, 64, 64, tid);
        if (tid < BD) rE = p.ws.EGL[u * BD + tid];
        fetch_tile<VBT>(rU, (const T*)p.ws.Um + u * 64 * BD + vcol0, BD, 64, tid);
    };
    if (sq.nc > 0) fetch(0);
    for (int64_t ic = 0; ic < sq.nc; ++ic) {
        const int64_t tok0 = sq.bos + ic * CH;
        const int valid = (int)min((int64_t)CH, sq.len - ic * CH);
        put_tile<BD>(sW, P128, rW, tid);
        put_tile<BD>(sKG, P128, rKG, tid);
        put_tile<BD>(sQG, P128, rQG, tid);
        put_tile<CH>(sP, P64, rP, tid);
        put_tile<VBT>(sU, PV, rU, tid);
        if (tid < BD) sE[tid] = rE;
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const V4 s4 = pack4<T>(S[a2][b]);
                *(V4*)(sS + (16 * (2 * w + a2) + c16) * PV + 16 * b + 4 * g) = s4;
                if (p.hs) *(V4*)((T*)p.hs + (((sq.cbase + ic) * p.HV + hv) * BD + 16 * (2 * w + a2) + c16) * BD + vcol0 + 16 * b + 4 * g) = s4;
            }
        lds_barrier();
        if (ic + 1 < sq.nc) fetch(ic + 1);
        f32x4 oacc[NB];
        {
            // v_new^T and (qg S)^T tiles: value columns on the rows, this wave's 16 tokens on the columns
            const int i = 16 * w + c16;
            V8 wf[4], qf[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) { wf[s] = frag_rows(sW, P128, 16 * w, 32 * s, lane); qf[s] = frag_rows(sQG, P128, 16 * w, 32 * s, lane); }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                f32x4 acc = ZERO4;
                oacc[b] = ZERO4;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const V8 fs = frag_cols(sS, PV, 32 * s, 16 * b, lane);
                    acc = Mma<T>::run(fs, wf[s], acc);
                    oacc[b] = Mma<T>::run(fs, qf[s], oacc[b]);
                }
                const V4 u4 = *(const V4*)(sU + i * PV + 16 * b + 4 * g);
                f32x4 vn;
#pragma unroll
                for (int r = 0; r < 4; ++r) vn[r] = (float)u4[r] - acc[r];
                *(V4*)(sVn + i * PV + 16 * b + 4 * g) = pack4<T>(vn);
            }
        }
        lds_barrier();
        {
            // o += P v_new;  S <- diag(e^Gam_last) S + kg^T v_new
            const int i = 16 * w + c16;
            V8 pf[2], kf[2][2];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                pf[s] = frag_rows(sP, P64, 16 * w, 32 * s, lane);
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2) kf[a2][s] = frag_cols(sKG, P128, 32 * s, 16 * (2 * w + a2), lane);
            }
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2) {
                const float e = sE[16 * (2 * w + a2) + c16];
#pragma unroll
                for (int b = 0; b < NB; ++b) S[a2][b] *= e;
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const V8 fv = frag_cols(sVn, PV, 32 * s, 16 * b, lane);
                    if (32 * s <= 16 * w + 15) oacc[b] = Mma<T>::run(fv, pf[s], oacc[b]);      // P[i][j] = 0 for j > i
#pragma unroll
                    for (int a2 = 0; a2 < 2; ++a2) S[a2][b] = Mma<T>::run(fv, kf[a2][s], S[a2][b]);
                }
                *(V4*)(sO + i * PV + 16 * b + 4 * g) = pack4<T>(oacc[b]);
            }
        }
        lds_barrier();
        copy_rows_out<64, VBT, 256>((T*)p.o + (tok0 * p.HV + hv) * BD + vcol0, (int64_t)p.HV * BD, sO, PV, tid, valid);
    }
    if (p.ht) {
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int kk = 16 * (2 * w + a2) + c16;
                *(f32x4*)(p.ht + ((n * p.HV + hv) * BD + kk) * BD + vcol0 + 16 * b + 4 * g) = S[a2][b];
            }
    }
}

template <typename T>
static int launch_kda(const KdaParams& p, int64_t num_chunks, hipStream_t stream, bool comba = false) {
    const int64_t runs1 = p.N * p.HV;
    const int vbt = runs1 <= 64 ? 32 : runs1 <= 128 ? 64 : 128;
    const unsigned units = (unsigned)(num_chunks * p.HV), runs = (unsigned)((runs1 + 7) / 8 * 8 * (BD / vbt));
    struct K { const void* f; size_t smem; const char* name; unsigned grid; };
    K scan;
    if (vbt == 32) scan = {(const void*)gdn_kda_scan_kernel<T, 32>, kda_scan_smem<32>(), "gdn_kda_scan_kernel", runs};
    else if (vbt == 64) scan = {(const void*)gdn_kda_scan_kernel<T, 64>, kda_scan_smem<64>(), "gdn_kda_scan_kernel", runs};
    else scan = {(const void*)gdn_kda_scan_kernel<T, 128>, kda_scan_smem<128>(), "gdn_kda_scan_kernel", runs};
    const K prep = comba ? K{(const void*)gdn_comba_prepare_kernel<T>, COMBA_PREP_SMEM, "gdn_comba_prepare_kernel", units < 512u ? units : 512u}
                         : K{(const void*)gdn_kda_prepare_kernel<T>, KDA_PREP_SMEM, "gdn_kda_prepare_kernel", units < 512u ? units : 512u};
    const K ks[2] = {prep, scan};
    for (int i = 0; i < 2; ++i) {
        if (int rc = ensure_dynamic_smem_for(ks[i].f, ks[i].smem, ks[i].name)) return rc;
        int64_t nunits = units;
        void* args[] = {(void*)&p, (void*)&nunits};             // (the prepare kernel walks over the units and takes their number)
        if (hipLaunchKernel(ks[i].f, dim3(ks[i].grid), dim3(256), args, ks[i].smem, stream) != hipSuccess) return check_launch(ks[i].name);
        if (int rc = check_launch(ks[i].name)) return rc;
    }
    return GDN_OK;
}


int launch_kda_prepare(const KdaParams& p, int64_t num_chunks, int qkv_dtype, hipStream_t stream) {
    const unsigned units = (unsigned)(num_chunks * p.HV);
    const void* f = qkv_dtype == GDN_DTYPE_BF16 ? (const void*)gdn_kda_prepare_kernel<bf16_t> : (const void*)gdn_kda_prepare_kernel<f16_t>;
    if (int rc = ensure_dynamic_smem_for(f, KDA_PREP_SMEM, "gdn_kda_prepare_kernel")) return rc;
    int64_t nunits = units;
    void* args[] = {(void*)&p, (void*)&nunits};
    if (hipLaunchKernel(f, dim3(units < 512u ? units : 512u), dim3(256), args, KDA_PREP_SMEM, stream) != hipSuccess) return check_launch("gdn_kda_prepare_kernel");
    return check_launch("gdn_kda_prepare_kernel");
}

// checks shared by the two entry points
static int check_shapes(const char* who, int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V, int64_t N, int64_t num_chunks,
                        const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets, int qkv_dtype, uint32_t flags, uint32_t known) {
    GDN_CHECK_ARG(B >= 1 && T >= 0 && H >= 1 && HV >= 1 && N >= 1 && num_chunks >= 0, GDN_ERR_INVALID, "%s: bad dimension", who);
    GDN_CHECK_ARG(HV % H == 0, GDN_ERR_INVALID, "%s: HV=%lld not divisible by H=%lld", who, (long long)HV, (long long)H);
    GDN_CHECK_ARG(K == BD && V == BD, GDN_ERR_UNSUPPORTED, "%s: K = V = 128 only (got K=%lld V=%lld); pad smaller head dims with zeros",
                  who, (long long)K, (long long)V);
    GDN_CHECK_ARG(qkv_dtype == GDN_DTYPE_BF16 || qkv_dtype == GDN_DTYPE_F16, GDN_ERR_UNSUPPORTED, "%s: q/k/v must be bf16 or f16", who);
    GDN_CHECK_ARG((flags & ~known) == 0, GDN_ERR_UNSUPPORTED, "%s: unknown flag (the state layout is the caller's)", who);
    GDN_CHECK_ARG(HV <= 65535 && num_chunks * HV < (1ll << 31) && N * HV * 4 < (1ll << 31), GDN_ERR_UNSUPPORTED,
                  "%s: too many heads or chunks for one launch", who);
    if (cu_seqlens) {
        GDN_CHECK_ARG(B == 1, GDN_ERR_INVALID, "%s: with cu_seqlens B must be 1", who);
        GDN_CHECK_ARG((chunk_table || num_chunks == 0) && chunk_offsets, GDN_ERR_INVALID, "%s: packed input needs chunk_table and chunk_offsets", who);
    } else {
        GDN_CHECK_ARG(N == B, GDN_ERR_INVALID, "%s: without cu_seqlens N must equal B", who);
        GDN_CHECK_ARG(num_chunks == B * ((T + CH - 1) / CH), GDN_ERR_INVALID, "%s: num_chunks does not match B and T", who);
    }
    return GDN_OK;
}

}  // namespace gdn

extern "C" size_t gdn_chunk_kda_workspace_bytes(int64_t num_chunks, int64_t HV) {
    if (num_chunks < 0 || HV < 1) return 0;
    return gdn::kda_ws_layout(num_chunks * HV, nullptr, nullptr);
}

static int kda_fwd_entry(
    const char* who,
    const void* q, const void* k, const void* v, const float* g, const void* beta,
    const float* A_log, const float* dt_bias, float lower_bound, int gate_mode,
    const float* h0, float* ht, void* o, void* states,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    using namespace gdn;
    const uint32_t known = GDN_FLAG_CU_INT32 | GDN_FLAG_QK_L2NORM | GDN_FLAG_BETA_SIGMOID | GDN_FLAG_NEG_EIGVAL;
    if (int rc = check_shapes(who, B, T, H, HV, K, V, N, num_chunks, cu_seqlens, chunk_table, chunk_offsets, qkv_dtype, flags, known)) return rc;
    GDN_CHECK_ARG(gate_mode >= 0 && gate_mode <= 2, GDN_ERR_INVALID, "%s: gate_mode must be 0, 1 or 2", who);
    GDN_CHECK_ARG(gate_mode != 0 || (!A_log && !dt_bias), GDN_ERR_INVALID, "%s: A_log / dt_bias without a gate activation", who);
    GDN_CHECK_ARG(!(flags & GDN_FLAG_NEG_EIGVAL) || (flags & GDN_FLAG_BETA_SIGMOID), GDN_ERR_INVALID, "%s: GDN_FLAG_NEG_EIGVAL needs GDN_FLAG_BETA_SIGMOID", who);
    hipStream_t s = (hipStream_t)stream;
    if (T == 0 || num_chunks == 0) {
        if (ht) return launch_state_copy(h0, ht, N * HV * K * V, s);
        return GDN_OK;
    }
    GDN_CHECK_ARG(q && k && v && g && beta && o, GDN_ERR_INVALID, "%s: q, k, v, g, beta, o must not be NULL", who);
    for (const void* x : {q, k, v, (const void*)g, (const void*)h0, (const void*)ht, (const void*)o, (const void*)states})
        GDN_CHECK_ARG(((uintptr_t)x % 16) == 0, GDN_ERR_INVALID, "%s: tensors must be 16-byte aligned", who);
    GDN_CHECK_ARG(((uintptr_t)workspace % 256) == 0, GDN_ERR_INVALID, "%s: the workspace must be 256-byte aligned", who);
    KdaParams p;
    const size_t need = kda_ws_layout(num_chunks * HV, (char*)workspace, &p.ws);
    GDN_CHECK_ARG(workspace && workspace_bytes >= need, GDN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who,
                  need, workspace_bytes);
    p.q = q; p.k = k; p.v = v; p.g = g; p.beta = beta; p.pk = nullptr; p.gs = nullptr; p.A_log = A_log; p.gk_bias = dt_bias; p.gk_lower = lower_bound; p.gk_act = gate_mode;
    p.h0 = h0; p.ht = ht; p.o = o; p.hs = states;
    p.cu_seqlens = cu_seqlens; p.chunk_table = chunk_table; p.chunk_offsets = chunk_offsets;
    p.T = T; p.H = (int)H; p.HV = (int)HV; p.N = N; p.NT = (T + CH - 1) / CH;
    p.scale = scale; p.gb_dtype = gb_dtype; p.flags = flags;
    return qkv_dtype == GDN_DTYPE_BF16 ? launch_kda<bf16_t>(p, num_chunks, s) : launch_kda<f16_t>(p, num_chunks, s);
}

extern "C" int gdn_chunk_kda_fwd(
    const void* q, const void* k, const void* v, const float* g, const void* beta,
    const float* A_log, const float* dt_bias, float lower_bound, int gate_mode,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    return kda_fwd_entry("gdn_chunk_kda_fwd", q, k, v, g, beta, A_log, dt_bias, lower_bound, gate_mode, h0, ht, o, nullptr, cu_seqlens, chunk_table,
                         chunk_offsets, workspace, workspace_bytes, B, T, H, HV, K, V, N, num_chunks, scale, qkv_dtype, gb_dtype, flags, stream);
}

// ... and the state in front of every chunk, states [num_chunks][HV][K][V] in qkv_dtype (the reference's h with return_intermediate_states)
extern "C" int gdn_chunk_kda_fwd_states(
    const void* q, const void* k, const void* v, const float* g, const void* beta,
    const float* A_log, const float* dt_bias, float lower_bound, int gate_mode,
    const float* h0, float* ht, void* o, void* states,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    GDN_CHECK_ARG(states || T == 0 || num_chunks == 0, GDN_ERR_INVALID, "gdn_chunk_kda_fwd_states: states must not be NULL");
    return kda_fwd_entry("gdn_chunk_kda_fwd_states", q, k, v, g, beta, A_log, dt_bias, lower_bound, gate_mode, h0, ht, o, states, cu_seqlens, chunk_table,
                         chunk_offsets, workspace, workspace_bytes, B, T, H, HV, K, V, N, num_chunks, scale, qkv_dtype, gb_dtype, flags, stream);
}

extern "C" int gdn_chunk_comba_fwd(
    const void* q, const void* k, const void* v, const void* p_key, const void* g, const void* beta,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    using namespace gdn;
    const char* who = "gdn_chunk_comba_fwd";
    if (int rc = check_shapes(who, B, T, H, HV, K, V, N, num_chunks, cu_seqlens, chunk_table, chunk_offsets, qkv_dtype, flags,
                              GDN_FLAG_CU_INT32 | GDN_FLAG_QK_L2NORM)) return rc;
    GDN_CHECK_ARG(gb_dtype == GDN_DTYPE_F32 || gb_dtype == GDN_DTYPE_BF16 || gb_dtype == GDN_DTYPE_F16, GDN_ERR_UNSUPPORTED,
                  "%s: g and beta must be f32, bf16 or f16", who);
    hipStream_t s = (hipStream_t)stream;
    if (T == 0 || num_chunks == 0) {
        if (ht) return launch_state_copy(h0, ht, N * HV * K * V, s);
        return GDN_OK;
    }
    GDN_CHECK_ARG(q && k && v && p_key && g && beta && o, GDN_ERR_INVALID, "%s: q, k, v, p, g, beta, o must not be NULL", who);
    for (const void* x : {q, k, v, p_key, (const void*)h0, (const void*)ht, (const void*)o})
        GDN_CHECK_ARG(((uintptr_t)x % 16) == 0, GDN_ERR_INVALID, "%s: tensors must be 16-byte aligned", who);
    GDN_CHECK_ARG(((uintptr_t)workspace % 256) == 0, GDN_ERR_INVALID, "%s: the workspace must be 256-byte aligned", who);
    KdaParams p;
    const size_t need = kda_ws_layout(num_chunks * HV, (char*)workspace, &p.ws);
    GDN_CHECK_ARG(workspace && workspace_bytes >= need, GDN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who,
                  need, workspace_bytes);
    p.q = q; p.k = k; p.v = v; p.g = nullptr; p.beta = beta; p.pk = p_key; p.gs = g;
    p.A_log = nullptr; p.gk_bias = nullptr; p.gk_lower = 0.f; p.gk_act = 0;
    p.h0 = h0; p.ht = ht; p.o = o; p.hs = nullptr;
    p.cu_seqlens = cu_seqlens; p.chunk_table = chunk_table; p.chunk_offsets = chunk_offsets;
    p.T = T; p.H = (int)H; p.HV = (int)HV; p.N = N; p.NT = (T + CH - 1) / CH;
    p.scale = scale; p.gb_dtype = gb_dtype; p.flags = flags;
    return qkv_dtype == GDN_DTYPE_BF16 ? launch_kda<bf16_t>(p, num_chunks, s, true) : launch_kda<f16_t>(p, num_chunks, s, true);
}
