// Backward pass of the chunked KDA operator (the gated delta rule with a decay per key feature; K, V <= 128, zero-padded
// to 128 by the host).  Included by gdn_chunk_bwd.hip inside namespace gdn, after its types and its two scans, which serve this
// pass in their KDA form.  Replaces
// chunk_kda_bwd (fla/ops/kda/chunk_bwd.py): the forward's chunk-parallel kernel runs again (A, w, u, qg, kg, P and the
// running sums Gk of the log decays), then
//
//   state, dstate   as for the gated delta rule, with kg / qg in place of k / q and a decay per key feature
//   dqkw            per (chunk, v-head): dw = -dv_new S^T, dPs = scale tril(do v_new^T), and the parts of dq, dk, dGk
//                   that come through qg, kg and e^Gk_last
//   wy              per (chunk, v-head): back through w = A (beta k e^Gk), u = A (beta v), A = (I + diag(beta) M)^-1 and
//                   through the two matrices with a decay per pair and feature,
//                       M_ij = sum_d k_id k_jd e^(Gk_id - Gk_jd) (i > j),   P_ij = scale sum_d q_id k_jd e^(Gk_id - Gk_jd) (i >= j);
//                   dg = reverse cumulative sum of dGk over the chunk's tokens
//
// Pairs and features: with dL the gradient of diag(beta)^-1 L and dPs that of P / scale o mask,
//   row side   dq_i  += sum_j dPs_ij k_j e^(Gk_i - Gk_j),     rk_i = sum_j dL_ij k_j e^(Gk_i - Gk_j)  (dbeta_i += k_i . rk_i,  dk_i += beta_i rk_i)
//   col side   dk_j  += sum_i (dPs_ij q_i + dL_ij beta_i k_i) e^(Gk_i - Gk_j)
//   dGk_i += q_i dq_i + k_i (beta_i rk_i),   dGk_j -= k_j (col side)_j        (elementwise in the feature)
// The exponent splits into a factor of row i and one of row j around a reference row R that lies between them: blocks of 16
// rows, R = the row in front of i's block, e^(Gk_i - R) <= 1 on the results, e^(R - Gk_j) on the operand rows (<= 1 for earlier
// blocks; inside the diagonal block >= 1, which the operand type holds as long as the block's total decay stays above a
// bound - otherwise every pair of the diagonal block gets its own exponentials, as in the forward kernel and in the
// reference's sub-chunks of 16, fla/ops/kda/chunk_intra.py).  All of it runs on the matrix cores: per block of rows one
// operand tile k e^(R - Gk) for the row side, and for the column side one 32-deep step whose contraction index runs over the
// block's 16 rows twice (dPs^T against q e^(Gk - R), dL^T against beta k e^(Gk - R)).

template <typename T> struct SpanOk { static constexpr float value = -8.f; };       // f16: factors up to e^8
template <> struct SpanOk<bf16_t> { static constexpr float value = -80.f; };

// ---------------------------------------------------------------------------------------------
// dqkw, KDA
// ---------------------------------------------------------------------------------------------
constexpr size_t BWD_DQKW_KDA_SMEM = (5 * 64 * P128) * 2 + (64 * PG + BD) * 4;

template <typename T>
__global__ __launch_bounds__(256, 1) void gdn_bwd_dqkw_kda_kernel(BwdParams p, int64_t units) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    T* sDO = (T*)smem; T* sVn = sDO + 64 * P128; T* sDvn = sVn + 64 * P128; T* sK = sDvn + 64 * P128; T* sQ = sK + 64 * P128;
    float* sG = (float*)(sQ + 64 * P128); float* sSd = sG + 64 * PG;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;

    TileRegs<BD> rDO, rVn, rDvn, rK, rQ;
    V8 rS[2][4], rdS[2][4];
    f32x4 rG[8];
    auto fetch = [&](int64_t u) {
        const int hv = (int)(u % p.HV), hq = hv / (p.HV / p.H);
        const ChunkAt c = chunk_at(p, u / p.HV);
        fetch_tile<BD>(rDO, (const T*)p.dout + (c.tok0 * p.HV + hv) * BD, (int64_t)p.HV * BD, c.valid, tid);
        fetch_tile<BD>(rVn, (const T*)p.ws.Vn + u * 64 * BD, BD, 64, tid);
        fetch_tile<BD>(rDvn, (const T*)p.ws.dVn + u * 64 * BD, BD, 64, tid);
        const T* Hu = (const T*)p.ws.Hs + u * BD * BD;
        const T* dHu = (const T*)p.ws.dHs + u * BD * BD;
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int kk = 16 * (2 * w + a2) + c16;
                rS[a2][s] = *(const V8*)(Hu + kk * BD + 32 * s + 8 * g);
                rdS[a2][s] = *(const V8*)(dHu + kk * BD + 32 * s + 8 * g);
            }
        fetch_tile<BD>(rK, (const T*)p.k + (c.tok0 * p.H + hq) * BD, (int64_t)p.H * BD, c.valid, tid);
        fetch_tile<BD>(rQ, (const T*)p.q + (c.tok0 * p.H + hq) * BD, (int64_t)p.H * BD, c.valid, tid);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int idx = tid + 256 * i;
            rG[i] = *(const f32x4*)(p.ws.Gk + u * 64 * BD + (idx >> 5) * BD + (idx & 31) * 4);
        }
    };
    fetch(blockIdx.x);
    const int tid_outer = tid;
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
        int tid_opaque = tid_outer;                             // (see gdn_bwd_wy_kda_kernel)
        asm volatile("" : "+v"(tid_opaque));
        const int tid = tid_opaque, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
        const int hv = (int)(u % p.HV);
        const ChunkAt c = chunk_at(p, u / p.HV);
        put_tile<BD>(sDO, P128, rDO, tid);
        put_tile<BD>(sVn, P128, rVn, tid);
        put_tile<BD>(sDvn, P128, rDvn, tid);
        put_tile<BD>(sK, P128, rK, tid);
        put_tile<BD>(sQ, P128, rQ, tid);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int idx = tid + 256 * i;
            *(f32x4*)(sG + (idx >> 5) * PG + (idx & 31) * 4) = rG[i];
        }
        V8 sf[2][4], df[2][4];
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
            for (int s = 0; s < 4; ++s) { sf[a2][s] = rS[a2][s]; df[a2][s] = rdS[a2][s]; }
        lds_barrier();
        if (u + gridDim.x < units) fetch(u + gridDim.x);

        f32x4 G1[2][4], dKS[2][4], dWt[2][4], dPt[4];
        float sd[2] = {0.f, 0.f};
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
            for (int t = 0; t < 4; ++t) G1[a2][t] = dWt[a2][t] = dKS[a2][t] = ZERO4;
#pragma unroll
        for (int t = 0; t < 4; ++t) dPt[t] = ZERO4;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
                for (int e = 0; e < 8; ++e) sd[a2] += (float)sf[a2][s][e] * (float)df[a2][s][e];
            const V8 own = frag_rows(sDO, P128, 16 * w, 32 * s, lane);             // this wave's 16 token rows of do, for dP
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const V8 bdo = frag_rows(sDO, P128, 16 * t, 32 * s, lane), bdv = frag_rows(sDvn, P128, 16 * t, 32 * s, lane),
                         bvn = frag_rows(sVn, P128, 16 * t, 32 * s, lane);
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2) {
                    G1[a2][t] = Mma<T>::run(sf[a2][s], bdo, G1[a2][t]);
                    dWt[a2][t] = Mma<T>::run(sf[a2][s], bdv, dWt[a2][t]);
                    dKS[a2][t] = Mma<T>::run(df[a2][s], bvn, dKS[a2][t]);
                }
                if (t <= w) dPt[t] = Mma<T>::run(own, bvn, dPt[t]);
            }
        }
        {
            T* dWu = (T*)p.ws.dWm + u * 64 * BD;
            T* dPu = (T*)p.ws.dPs + u * 64 * 64;
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    *(V4*)(dWu + (16 * t + c16) * BD + 16 * (2 * w + a2) + 4 * g) = pack4<T>(-dWt[a2][t]);
            // dPs = scale tril(do v_new^T): lane holds column j = 16tj + c16, rows 16w + 4g + r
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                const int j = 16 * tj + c16;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    dPu[i * 64 + j] = (T)(i >= j ? p.scale * dPt[tj][r] : 0.f);
                }
            }
            // <S, dS> per key feature: the decay e^Gk_last of the state
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2) {
                const float x = sum_over_g(sd[a2]);
                if (g == 0) sSd[16 * (2 * w + a2) + c16] = x;
            }
        }
        lds_barrier();
        f32x4 glsum[2] = {ZERO4, ZERO4}, dG63[2] = {ZERO4, ZERO4};
        float* dGu = p.ws.dGk + u * 64 * BD;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int x = 16 * t + c16;
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2) {
                const int n16 = 16 * (2 * w + a2);
                const f32x4 Gx = *(const f32x4*)(sG + x * PG + n16 + 4 * g), Gl = *(const f32x4*)(sG + 63 * PG + n16 + 4 * g);
                const V4 q4 = *(const V4*)(sQ + x * P128 + n16 + 4 * g), k4 = *(const V4*)(sK + x * P128 + n16 + 4 * g);
                f32x4 dq, dk, dG;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    dq[r] = G1[a2][t][r] * (p.scale * __expf(Gx[r]));
                    dk[r] = dKS[a2][t][r] * __expf(Gl[r] - Gx[r]);
                    const float kdk = (float)k4[r] * dk[r];
                    glsum[a2][r] += kdk;
                    dG[r] = (float)q4[r] * dq[r] - kdk;
                }
                if (x < c.valid) {
                    *(V4*)((T*)p.dq + ((c.tok0 + x) * p.HV + hv) * BD + n16 + 4 * g) = pack4<T>(dq);
                    *(V4*)((T*)p.dk + ((c.tok0 + x) * p.HV + hv) * BD + n16 + 4 * g) = pack4<T>(dk);
                }
                if (t == 3 && c16 == 15) dG63[a2] = dG;         // the chunk's last row also takes what goes through e^Gk_last
                else *(f32x4*)(dGu + x * BD + n16 + 4 * g) = dG;
            }
        }
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2) {
            const int n16 = 16 * (2 * w + a2);
            f32x4 tot;
#pragma unroll
            for (int r = 0; r < 4; ++r) tot[r] = sum_over_c16(glsum[a2][r]);
            if (c16 == 15) {
                const f32x4 Gl = *(const f32x4*)(sG + 63 * PG + n16 + 4 * g), sdv = *(const f32x4*)(sSd + n16 + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) dG63[a2][r] += tot[r] + __expf(Gl[r]) * sdv[r];
                *(f32x4*)(dGu + 63 * BD + n16 + 4 * g) = dG63[a2];
            }
        }
        lds_barrier();
    }
}

// ---------------------------------------------------------------------------------------------
// wy, KDA
// ---------------------------------------------------------------------------------------------
constexpr size_t BWD_WY_KDA_SMEM = (5 * 64 * P128 + 4 * 64 * P64) * 2 + (64 * PG + 64 + 256) * 4;

template <typename T>
__global__ __launch_bounds__(256, 1) void gdn_bwd_wy_kda_kernel(BwdParams p, int64_t units) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    T* sDvn = (T*)smem; T* sV = sDvn + 64 * P128; T* sDW = sV + 64 * P128; T* sK = sDW + 64 * P128; T* sKp = sK + 64 * P128;
    T* sA = sKp + 64 * P128; T* sM1 = sA + 64 * P64; T* sM2 = sM1 + 64 * P64; T* sDPs = sM2 + 64 * P64;
    float* sG = (float*)(sDPs + 64 * P64); float* sBeta = sG + 64 * PG; float* sDb = sBeta + 64;
    T* sQ = sDvn;                                               // the rows of q take the place of dv_new's once those are done with
    T* sT = sV;                                                 // operand rows k e^(R - Gk) of the current block, in v's place
    T* sOp = sDW;                                               // 32 operand rows of the column side, in dw's place
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    auto feat = [&](int a) { return 16 * (2 * w + a); };        // first key feature of this wave's tile a

    TileRegs<BD> rDvn, rV, rDW, rK, rQ;
    TileRegs<CH> rA, rDPs;
    f32x4 rG[8];
    uint32_t rBeta = 0;                                          // (raw bits: converted when the unit's turn comes)
    auto fetch = [&](int64_t u) {
        const int hv = (int)(u % p.HV), hq = hv / (p.HV / p.H);
        const ChunkAt c = chunk_at(p, u / p.HV);
        fetch_tile<BD>(rDvn, (const T*)p.ws.dVn + u * 64 * BD, BD, 64, tid);
        fetch_tile<BD>(rV, (const T*)p.v + (c.tok0 * p.HV + hv) * BD, (int64_t)p.HV * BD, c.valid, tid);
        fetch_tile<CH>(rA, (const T*)p.ws.Am + u * 64 * 64, 64, 64, tid);
        fetch_tile<BD>(rDW, (const T*)p.ws.dWm + u * 64 * BD, BD, 64, tid);
        fetch_tile<BD>(rK, (const T*)p.k + (c.tok0 * p.H + hq) * BD, (int64_t)p.H * BD, c.valid, tid);
        fetch_tile<CH>(rDPs, (const T*)p.ws.dPs + u * 64 * 64, 64, 64, tid);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int idx = tid + 256 * i;
            rG[i] = *(const f32x4*)(p.ws.Gk + u * 64 * BD + (idx >> 5) * BD + (idx & 31) * 4);
        }
        if (tid < 64) rBeta = tid < c.valid ? load_scalar_bits(p.beta, (c.tok0 + tid) * p.HV + hv, p.gb_dtype) : 0;
    };
    fetch(blockIdx.x);
    const int tid_outer = tid;
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
        // (everything derived from the lane number is derived again per unit from a copy the compiler cannot see through:
        // hoisted out of this loop, the addresses of its unrolled body would fill the register file and spill)
        int tid_opaque = tid_outer;
        asm volatile("" : "+v"(tid_opaque));
        const int tid = tid_opaque, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
        auto feat = [&](int a) { return 16 * (2 * w + a); };
        const int hv = (int)(u % p.HV), hq = hv / (p.HV / p.H);
        const ChunkAt c = chunk_at(p, u / p.HV);
        put_tile<BD>(sDvn, P128, rDvn, tid);
        put_tile<BD>(sV, P128, rV, tid);
        put_tile<CH>(sA, P64, rA, tid);
        put_tile<BD>(sDW, P128, rDW, tid);
        put_tile<BD>(sK, P128, rK, tid);
        put_tile<CH>(sDPs, P64, rDPs, tid);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int idx = tid + 256 * i;
            *(f32x4*)(sG + (idx >> 5) * PG + (idx & 31) * 4) = rG[i];
        }
        if (tid < 64) sBeta[tid] = scalar_of_bits(rBeta, p.gb_dtype);
        sDb[tid] = 0.f;
        lds_barrier();
        // this unit's rows of q (wanted late, no room for them in LDS yet) and what the previous kernel left of dGk
        fetch_tile<BD>(rQ, (const T*)p.q + (c.tok0 * p.H + hq) * BD, (int64_t)p.H * BD, c.valid, tid);
        f32x4 dG[2][4];
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
            for (int t = 0; t < 4; ++t) dG[a2][t] = *(const f32x4*)(p.ws.dGk + u * 64 * BD + (16 * t + c16) * BD + feat(a2) + 4 * g);
        // k e^Gk, the factor of w
        for (int idx = tid; idx < 64 * 16; idx += 256) {
            const int row = idx >> 4, pc = idx & 15;
            V8 kx = *(const V8*)(sK + row * P128 + pc * 8);
            const float* gi = sG + row * PG + pc * 8;
#pragma unroll
            for (int e = 0; e < 8; ++e) kx[e] = (T)((float)kx[e] * __expf(gi[e]));
            *(V8*)(sKp + row * P128 + pc * 8) = kx;
        }
        // the decay across each block of 16 rows, the strongest over the features: decides how the diagonal blocks are treated
        bool ok[4];
        {
            float span[4];
#pragma unroll
            for (int ti = 0; ti < 4; ++ti) {
                span[ti] = 0.f;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int col = lane + 64 * h;
                    span[ti] = fminf(span[ti], sG[(16 * ti + 15) * PG + col] - (ti > 0 ? sG[(16 * ti - 1) * PG + col] : 0.f));
                }
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) span[ti] = fminf(span[ti], __shfl_xor(span[ti], off, 64));
                ok[ti] = span[ti] >= SpanOk<T>::value;
            }
        }
        lds_barrier();

        // dX = du v^T + dw (k e^Gk)^T (this wave's 16 rows i; lane: column j, rows 4g + r);  dA = stril(dX diag(beta))
        {
            V8 fa[4], fw[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                fa[s] = frag_rows(sDvn, P128, 16 * w, 32 * s, lane);
                fw[s] = frag_rows(sDW, P128, 16 * w, 32 * s, lane);
            }
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                f32x4 dX = ZERO4;
                if (tj <= w) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        dX = Mma<T>::run(fa[s], frag_rows(sV, P128, 16 * tj, 32 * s, lane), dX);
                        dX = Mma<T>::run(fw[s], frag_rows(sKp, P128, 16 * tj, 32 * s, lane), dX);
                    }
                }
                const int j = 16 * tj + c16;
                const float bj = sBeta[j];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    sM1[i * P64 + j] = (T)(i > j ? dX[r] * bj : 0.f);
                }
            }
        }
        // dv = beta (A^T du);  d(k e^Gk) = beta (A^T dw): into dk, dbeta, dGk
        f32x4 dk[2][4];
        {
            V8 fA[4][2];                                        // A^T operand of token tile t, step s (zero where A is)
            float bj[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int s = 0; s < 2; ++s)
                    if (32 * s + 31 >= 16 * t) fA[t][s] = frag_cols(sA, P64, 32 * s, 16 * t, lane);
                bj[t] = sBeta[16 * t + c16];
            }
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2) {
                const int n16 = feat(a2);
                V8 fdv[2], fdw[2];
#pragma unroll
                for (int s = 0; s < 2; ++s) { fdv[s] = frag_cols(sDvn, P128, 32 * s, n16, lane); fdw[s] = frag_cols(sDW, P128, 32 * s, n16, lane); }
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    f32x4 av = ZERO4, ak = ZERO4;
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        if (32 * s + 31 < 16 * t) continue;     // A[i][j] = 0 for i < j
                        av = Mma<T>::run(fdv[s], fA[t][s], av);
                        ak = Mma<T>::run(fdw[s], fA[t][s], ak);
                    }
                    const int j = 16 * t + c16;
                    const V4 v4 = *(const V4*)(sV + j * P128 + n16 + 4 * g), kp4 = *(const V4*)(sKp + j * P128 + n16 + 4 * g);
                    const f32x4 Gj = *(const f32x4*)(sG + j * PG + n16 + 4 * g);
                    float dbv = 0.f;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        dbv += av[r] * (float)v4[r] + ak[r] * (float)kp4[r];
                        dk[a2][t][r] = ak[r] * (bj[t] * __expf(Gj[r]));
                        dG[a2][t][r] += bj[t] * (float)kp4[r] * ak[r];
                    }
                    dbv = sum_over_g(dbv);
                    if (g == 0) atomicAdd(&sDb[64 * w + j], dbv);
                    if (j < c.valid) *(V4*)((T*)p.dv + ((c.tok0 + j) * p.HV + hv) * BD + n16 + 4 * g) = pack4<T>(av * bj[t]);
                }
            }
        }
        lds_barrier();
        put_tile<BD>(sQ, P128, rQ, tid);                        // (dv_new's rows are done with)
        // Y = dA A^T
        {
            V8 fd[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) fd[s] = frag_rows(sM1, P64, 16 * w, 32 * s, lane);
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) {
                f32x4 acc = ZERO4;
#pragma unroll
                for (int s = 0; s < 2; ++s) acc = Mma<T>::run(fd[s], frag_rows(sA, P64, 16 * tl, 32 * s, lane), acc);
                const int l = 16 * tl + c16;
#pragma unroll
                for (int r = 0; r < 4; ++r) sM2[(16 * w + 4 * g + r) * P64 + l] = (T)acc[r];
            }
        }
        lds_barrier();
        // dL = -stril(A^T Y): the gradient of stril(M) once its rows are scaled by beta
        {
            V8 fAt[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) fAt[s] = frag_cols(sA, P64, 32 * s, 16 * w, lane);
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) {
                f32x4 acc = ZERO4;
                if (tl <= w) {
#pragma unroll
                    for (int s = 0; s < 2; ++s) acc = Mma<T>::run(fAt[s], frag_cols(sM2, P64, 32 * s, 16 * tl, lane), acc);
                }
                const int l = 16 * tl + c16;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    sM1[i * P64 + l] = (T)(i > l ? -acc[r] : 0.f);
                }
            }
        }
        lds_barrier();
        // (the next unit's tiles are requested here, not at the top of the unit: there the requests queue behind the last unit's stores)
        if (u + gridDim.x < units) fetch(u + gridDim.x);
        // the two matrices with a decay per pair and feature, a block of 16 rows at a time
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
            const int nj = 16 * (ti + 1), njp = (nj + 31) & ~31;
            const float* sR = sG + (16 * ti - 1) * PG;          // the reference row (zeros for the first block)
            for (int idx = tid; idx < njp * 16; idx += 256) {
                const int row = idx >> 4, pc = idx & 15;
                V8 out;
#pragma unroll
                for (int e = 0; e < 8; ++e) out[e] = (T)0.f;
                if (row < nj && (ok[ti] || row < 16 * ti)) {
                    const V8 kx = *(const V8*)(sK + row * P128 + pc * 8);
                    const float* gj = sG + row * PG + pc * 8;
#pragma unroll
                    for (int e = 0; e < 8; ++e) out[e] = (T)((float)kx[e] * __expf((ti > 0 ? sR[pc * 8 + e] : 0.f) - gj[e]));
                }
                *(V8*)(sT + row * P128 + pc * 8) = out;
            }
            for (int idx = tid; idx < 32 * 16; idx += 256) {
                const int row = idx >> 4, pc = idx & 15, i = 16 * ti + (row & 15);
                const V8 x = *(const V8*)((row < 16 ? sQ : sK) + i * P128 + pc * 8);
                const float* gi = sG + i * PG + pc * 8;
                const float m = row < 16 ? 1.f : sBeta[i];
                V8 out;
#pragma unroll
                for (int e = 0; e < 8; ++e) out[e] = (T)((float)x[e] * (m * __expf(gi[e] - (ti > 0 ? sR[pc * 8 + e] : 0.f))));
                *(V8*)(sOp + row * P128 + pc * 8) = out;
            }
            const int x = 16 * ti + c16;
            V4 dq_old[2];                                       // what the previous kernel left in dq, at this lane's places
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2) {
                dq_old[a2] = V4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
                if (x < c.valid) dq_old[a2] = *(const V4*)((const T*)p.dq + ((c.tok0 + x) * p.HV + hv) * BD + feat(a2) + 4 * g);
            }
            lds_barrier();
            const float bx = sBeta[x];
            f32x4 rq[2] = {ZERO4, ZERO4}, rk[2] = {ZERO4, ZERO4};     // (rk: before the row's beta)
#pragma unroll
            for (int s = 0; 32 * s < njp; ++s) {
                const V8 bq = frag_rows(sDPs, P64, 16 * ti, 32 * s, lane), bl = frag_rows(sM1, P64, 16 * ti, 32 * s, lane);
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2) {
                    const V8 fa = frag_cols(sT, P128, 32 * s, feat(a2), lane);
                    rq[a2] = Mma<T>::run(fa, bq, rq[a2]);
                    rk[a2] = Mma<T>::run(fa, bl, rk[a2]);
                }
            }
            // dGk takes every product dPs_ij (q_i f_i) (k_j e^(R - Gk_j)) twice, once with each sign (row i, column j), and
            // the sums down the columns leave the difference: both sides form it from the same rounded operands
            f32x4 R4[2], Gx4[2];
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2) {
                R4[a2] = ti > 0 ? *(const f32x4*)(sR + feat(a2) + 4 * g) : ZERO4;
                Gx4[a2] = *(const f32x4*)(sG + x * PG + feat(a2) + 4 * g);
                const V4 qf4 = *(const V4*)(sOp + c16 * P128 + feat(a2) + 4 * g), kf4 = *(const V4*)(sOp + (16 + c16) * P128 + feat(a2) + 4 * g);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    dG[a2][ti][r] += (float)qf4[r] * rq[a2][r] + (float)kf4[r] * rk[a2][r];
                    const float f = __expf(Gx4[a2][r] - R4[a2][r]);
                    rq[a2][r] *= f; rk[a2][r] *= f;
                }
            }
            if (!ok[ti]) {
                // the diagonal block pair by pair: row side for this lane's token x
#pragma unroll 1
                for (int jl = 0; jl < 16; ++jl) {
                    const int j = 16 * ti + jl;
                    if (j > x) continue;
                    const float a = (float)sDPs[x * P64 + j], b = (float)sM1[x * P64 + j];
#pragma unroll
                    for (int a2 = 0; a2 < 2; ++a2) {
                        const V4 k4 = *(const V4*)(sK + j * P128 + feat(a2) + 4 * g);
                        const V4 qx4 = *(const V4*)(sQ + x * P128 + feat(a2) + 4 * g), kx4 = *(const V4*)(sK + x * P128 + feat(a2) + 4 * g);
                        const f32x4 Gj = *(const f32x4*)(sG + j * PG + feat(a2) + 4 * g);
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const float kd = (float)k4[r] * __expf(Gx4[a2][r] - Gj[r]);
                            rq[a2][r] += a * kd; rk[a2][r] += b * kd;
                            dG[a2][ti][r] += ((float)qx4[r] * a + (float)kx4[r] * (bx * b)) * kd;
                        }
                    }
                }
            }
            float dbx = 0.f;
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2) {
                const V4 k4 = *(const V4*)(sK + x * P128 + feat(a2) + 4 * g);
                f32x4 dq;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    dbx += (float)k4[r] * rk[a2][r];
                    dk[a2][ti][r] += bx * rk[a2][r];
                    dq[r] = (float)dq_old[a2][r] + rq[a2][r];
                }
                if (x < c.valid) *(V4*)((T*)p.dq + ((c.tok0 + x) * p.HV + hv) * BD + feat(a2) + 4 * g) = pack4<T>(dq);
            }
            dbx = sum_over_g(dbx);
            if (g == 0) atomicAdd(&sDb[64 * w + x], dbx);
            // column side: the block's rows against the columns of this and the earlier blocks
#pragma unroll
            for (int tj = 0; tj <= ti; ++tj) {
                if (tj == ti && !ok[ti]) continue;
                const V8 bm = frag_cols(g < 2 ? sDPs : sM1, P64, g < 2 ? 16 * ti : 16 * ti - 16, 16 * tj, lane);
                const int xj = 16 * tj + c16;
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2) {
                    f32x4 col = Mma<T>::run(frag_cols(sOp, P128, 0, feat(a2), lane), bm, ZERO4);
                    const f32x4 Gj = *(const f32x4*)(sG + xj * PG + feat(a2) + 4 * g);
                    const V4 kt4 = *(const V4*)(sT + xj * P128 + feat(a2) + 4 * g);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        dk[a2][tj][r] += col[r] * __expf(R4[a2][r] - Gj[r]);
                        dG[a2][tj][r] -= (float)kt4[r] * col[r];
                    }
                }
            }
            if (!ok[ti]) {
                // ... and the column side for this lane's token x
#pragma unroll 1
                for (int il = 0; il < 16; ++il) {
                    const int i = 16 * ti + il;
                    if (i < x) continue;
                    const float a = (float)sDPs[i * P64 + x], b = (float)sM1[i * P64 + x] * sBeta[i];
#pragma unroll
                    for (int a2 = 0; a2 < 2; ++a2) {
                        const V4 q4 = *(const V4*)(sQ + i * P128 + feat(a2) + 4 * g), k4 = *(const V4*)(sK + i * P128 + feat(a2) + 4 * g);
                        const V4 kx4 = *(const V4*)(sK + x * P128 + feat(a2) + 4 * g);
                        const f32x4 Gi = *(const f32x4*)(sG + i * PG + feat(a2) + 4 * g);
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const float cv = (a * (float)q4[r] + b * (float)k4[r]) * __expf(Gi[r] - Gx4[a2][r]);
                            dk[a2][ti][r] += cv;
                            dG[a2][ti][r] -= (float)kx4[r] * cv;
                        }
                    }
                }
            }
            lds_barrier();
        }
        // dk on top of what the previous kernel left;  dGk into LDS for the sums down the columns
        {
            V4 dk_old[2][4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2) {
                    const int x = 16 * t + c16;
                    dk_old[a2][t] = V4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
                    if (x < c.valid) dk_old[a2][t] = *(const V4*)((const T*)p.dk + ((c.tok0 + x) * p.HV + hv) * BD + feat(a2) + 4 * g);
                }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int x = 16 * t + c16;
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2) {
                    f32x4 acc = dk[a2][t];
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[r] += (float)dk_old[a2][t][r];
                    *(V4*)(sT + x * P128 + feat(a2) + 4 * g) = pack4<T>(acc);     // (the operand rows are done with: dk leaves from here as whole rows)
                    *(f32x4*)(sG + x * PG + feat(a2) + 4 * g) = dG[a2][t];
                }
            }
        }
        lds_barrier();
        copy_rows_out<64, BD, 256>((T*)p.dk + (c.tok0 * p.HV + hv) * BD, (int64_t)p.HV * BD, sT, P128, tid, c.valid);
        {
            // dg = reverse cumulative sum of dGk: a thread per key feature and half of the rows
            const int f = tid & 127, half = tid >> 7;
            float run = 0.f;
            if (half == 0) {
#pragma unroll 8
                for (int r = 63; r >= 32; --r) run += sG[r * PG + f];
            }
            float* out = p.dgk + ((c.tok0 + 32 * half) * p.HV + hv) * BD + f;
#pragma unroll 8
            for (int r = 31; r >= 0; --r) {
                run += sG[(32 * half + r) * PG + f];
                if (32 * half + r < c.valid) out[(int64_t)r * p.HV * BD] = run;
            }
            if (tid < 64 && tid < c.valid)
                p.dbeta[(c.tok0 + tid) * p.HV + hv] = (sDb[tid] + sDb[64 + tid]) + (sDb[128 + tid] + sDb[192 + tid]);
        }
        lds_barrier();
    }
}

template <typename T>
static int launch_bwd_kda(const BwdParams& p, const KdaParams& kp, int64_t num_chunks, int qkv_dtype, hipStream_t stream) {
    if (int rc = launch_kda_prepare(kp, num_chunks, qkv_dtype, stream)) return rc;
    const int64_t runs1 = p.N * p.HV;
    const unsigned units = (unsigned)(num_chunks * p.HV);
    auto runs = [&](int v) { return (unsigned)((runs1 + 7) / 8 * 8 * (BD / v)); };
    struct K { const void* f; size_t smem; const char* name; unsigned grid, threads; };
    K state, dstate;
    int64_t nstate = 0;
    if (runs1 <= 128) {
        // both scans in one launch, every workgroup with a CU to itself, as many value columns each as that allows
        const int va = runs1 <= 32 ? 32 : runs1 <= 64 ? 64 : 128;
        nstate = runs(va);
        if (va == 32) state = {(const void*)gdn_bwd_scans_apart_kernel<T, 32, 1, true>, bwd_scans_apart_smem<32, 1>(), "gdn_bwd_scans_apart_kernel", 2 * runs(32), 256};
        else if (va == 64) state = {(const void*)gdn_bwd_scans_apart_kernel<T, 64, 1, true>, bwd_scans_apart_smem<64, 1>(), "gdn_bwd_scans_apart_kernel", 2 * runs(64), 256};
        else state = {(const void*)gdn_bwd_scans_apart_kernel<T, 128, 1, true>, bwd_scans_apart_smem<128, 1>(), "gdn_bwd_scans_apart_kernel", 2 * runs(128), 512};
        dstate = {nullptr, 0, "", 0, 0};
    } else {
        state = {(const void*)gdn_bwd_state_kernel<T, 128, 1, true>, bwd_state_smem<128, 1>(), "gdn_bwd_state_kernel", runs(128), 512};
        dstate = {(const void*)gdn_bwd_dstate_kernel<T, 128, 1, true>, bwd_dstate_smem<128, 1>(), "gdn_bwd_dstate_kernel", runs(128), 512};
    }
    const K ks[4] = {
        state, dstate,
        {(const void*)gdn_bwd_dqkw_kda_kernel<T>, BWD_DQKW_KDA_SMEM, "gdn_bwd_dqkw_kda_kernel", units < 256u ? units : 256u, 256},
        {(const void*)gdn_bwd_wy_kda_kernel<T>, BWD_WY_KDA_SMEM, "gdn_bwd_wy_kda_kernel", units < 256u ? units : 256u, 256},
    };
    int64_t nunits = units;
    for (int i = 0; i < 4; ++i) {
        if (ks[i].grid == 0) continue;
        if (int rc = ensure_dynamic_smem_for(ks[i].f, ks[i].smem, ks[i].name)) return rc;
        void* args[] = {(void*)&p, i == 0 && nstate ? (void*)&nstate : (void*)&nunits};
        if (hipLaunchKernel(ks[i].f, dim3(ks[i].grid), dim3(ks[i].threads), args, ks[i].smem, stream) != hipSuccess) return check_launch(ks[i].name);
        if (int rc = check_launch(ks[i].name)) return rc;
    }
    return GDN_OK;
}
