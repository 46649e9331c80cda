// Backward pass of the chunked gated delta rule (gfx950, 64-token chunks, 128 or 256 key features, 128 value columns; the host pads other head dims).
// Replaces the reference's backward pipeline fla/ops/gated_delta_rule/chunk.py:125-257 (recompute_w_u_fwd,
// chunk_gated_delta_rule_fwd_h, chunk_bwd_dv_local, chunk_gated_delta_rule_bwd_dhu, chunk_bwd_dqkwg, prepare_wy_repr_bwd,
// reverse chunk_local_cumsum) by five kernels:
//
//   prepare   per (chunk, v-head)      gam = cumsum(g), A = (I + diag(beta) stril(k k^T o D))^-1, w = A (beta e^gam k), u = A (beta v),
//                                      P^T with P = scale tril(q k^T o D);  D_ij = e^(gam_i - gam_j)
//   state     per (sequence, v-head, 32 value columns), chunks in order:   S_c (state in front of chunk c), v_new = u - w S_c
//   dstate    the same units, chunks in reverse order:   dS_c (gradient of the state behind chunk c),
//                                      dv_new = P^T do + (k e^(gam_last - gam)) dS_c,  dS <- e^gam_last dS + scale (q e^gam)^T do - w^T dv_new
//   dqkw      per (chunk, v-head)      dq, the parts of dk and dgam that come from the output and the state update, dw = -dv_new S^T
//   wy        per (chunk, v-head)      through w, u, A back to k, v, beta, gam; dg = reverse cumulative sum of dgam
//
// The comba operator (fla/ops/comba/chunk.py:92-178) predicts with a second key p and the state BEFORE the token's decay:
// with gam0 = gam - g its chunk form has A = (I + diag(beta) stril(p k^T o D0))^-1, D0_ij = e^(gam0_i - gam_j), and
// w = A (beta e^gam0 p); everything between w, u and the state is the gated delta rule's.  So the two scans and the dqkw
// kernel serve it unchanged, and `prepare` and `wy` have a COMBA form (one more tile: the rows of p; a second gradient,
// dgam0, whose reverse cumulative sum enters dg without its own token).
//
// All matrix products run on the matrix cores from row-major LDS tiles.  A product's two operands have the same register
// layout (lane (c16, g) holds index c16 and the 8 contraction indices 8g .. 8g+7 of a 32-wide step), so there are just two
// ways to fetch an operand fragment from a row-major tile: `frag_rows` (the contraction runs along a row: one 16-byte read)
// and `frag_cols` (the contraction runs down a column: two transposing LDS reads).  The result of run(a, b) holds, in lane
// (c16, g), column c16 (b's index) and rows 4g .. 4g+3 (a's index): whichever side carries the features gets them four in a
// row per lane, which is what an 8-byte store into a row-major [token][feature] array wants.
#include "gdn_chunk_kda.h"

namespace gdn {

// Per (chunk, v-head) unit, in separate arrays: gam [64] fp32, dgam [64] fp32 (partial, between the last two kernels), gam0 [64] fp32 (comba),
// A [64][64], P^T [64][64], w [64][KD], u -> v_new [64][128], S [KD][128] ([K][V]), dS [KD][128], dv_new [64][128],
// dw [64][KD], all in the operand type.
// The KDA operator (a decay per key feature) adds: Gk, the running sums of the log decays [64][128] fp32; QG = scale q e^Gk,
// KG = k e^(Gk_last - Gk) [64][128] and P [64][64] in the operand type, EGL = e^Gk_last [128] fp32 (all four as the forward's
// chunk-parallel kernel writes them); dPs = scale tril(do v_new^T) [64][64]; dGk [64][128] fp32 (partial, between the last two kernels).
// Um: u [64][128], read by the forward scan (which leaves v_new in Vn: a scan cut into time segments reads the u of chunks that belong
// to another workgroup, so it must not be overwritten); Bound: one float per unit, see gdn_chunk_common.h (WARM_LOG2).
struct BwdWs {
    float* Gam; float* Dgam; float* Gam0;
    void* Am; void* PT; void* Wm; void* Vn; void* Hs; void* dHs; void* dVn; void* dWm;
    float* Gk; void* QG; void* KG; void* Pm; float* EGL; void* dPs; float* dGk;
    void* Um; float* Bound;
};
inline size_t bwd_ws_layout(int64_t units, int64_t KD, char* base, BwdWs* ws) {
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += ws_align(bytes); return base ? (void*)(base + o) : nullptr; };
    const size_t u = (size_t)units;
    void* Gam = take(u * 64 * 4); void* Dgam = take(u * 64 * 4); void* Gam0 = take(u * 64 * 4);
    void* Am = take(u * 64 * 64 * 2); void* PT = take(u * 64 * 64 * 2);
    void* Wm = take(u * 64 * KD * 2); void* Vn = take(u * 64 * BD * 2);
    void* Hs = take(u * KD * BD * 2); void* dHs = take(u * KD * BD * 2);
    void* dVn = take(u * 64 * BD * 2); void* dWm = take(u * 64 * KD * 2);
    void* Um = take(u * 64 * BD * 2); void* Bound = take(u * 4);
    if (ws) *ws = BwdWs{(float*)Gam, (float*)Dgam, (float*)Gam0, Am, PT, Wm, Vn, Hs, dHs, dVn, dWm,
                        nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, Um, (float*)Bound};
    return off;
}
inline size_t kda_bwd_ws_layout(int64_t units, char* base, BwdWs* ws) {
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += ws_align(bytes); return base ? (void*)(base + o) : nullptr; };
    const size_t u = (size_t)units;
    void* Am = take(u * 64 * 64 * 2); void* Pm = take(u * 64 * 64 * 2); void* dPs = take(u * 64 * 64 * 2);
    void* Wm = take(u * 64 * BD * 2); void* Vn = take(u * 64 * BD * 2);
    void* QG = take(u * 64 * BD * 2); void* KG = take(u * 64 * BD * 2);
    void* Hs = take(u * BD * BD * 2); void* dHs = take(u * BD * BD * 2);
    void* dVn = take(u * 64 * BD * 2); void* dWm = take(u * 64 * BD * 2);
    void* Gk = take(u * 64 * BD * 4); void* dGk = take(u * 64 * BD * 4); void* EGL = take(u * BD * 4);
    if (ws) *ws = BwdWs{nullptr, nullptr, nullptr, Am, nullptr, Wm, Vn, Hs, dHs, dVn, dWm,
                        (float*)Gk, QG, KG, Pm, (float*)EGL, dPs, (float*)dGk, Vn, nullptr};       // (u and v_new share their place: whole sequences only)
    return off;
}

struct BwdParams {
    const void* q; const void* k; const void* v; const void* g; const void* beta;
    const float* h0; const void* dout; const float* dht;
    void* dq; void* dk; void* dv; float* dg; float* dbeta; float* dh0;
    const void* pk; void* dp;            // (comba) the second key, the one the prediction is made with, and its gradient
    float* dgk;                          // (KDA) gradient of the log decays [B,T,HV,128] fp32
    // The l2 normalisation of q and k taken in here (H == HV, one block of key features): the rows as the caller has them; q and k
    // above are then places in the workspace that the prepare kernel fills with the normalised rows, and these with the factors
    // [tokens,H] (fla/modules/l2norm.py:222-262); dq and dk come back as the gradients of the rows before the normalisation,
    // dx = (dy - y (y . dy)) rstd (fla/modules/l2norm.py:265-298).  NULL: q and k are what the recurrence uses.
    const void* q_raw; const void* k_raw; const void* pk_raw;    // (pk_raw, p_rstd: comba's second key, the same way)
    const float* q_rstd; const float* k_rstd; const float* p_rstd;
    const void* cu_seqlens; const void* chunk_table; const void* chunk_offsets;
    BwdWs ws;
    int64_t T; int H, HV; int64_t N; int64_t NT;
    float scale; int gb_dtype; uint32_t flags;
    // The two scans cut into `nseg` time segments of `seg_chunks` chunks (1: whole sequences): a segment starts from a zero state up
    // to `warm_cap` chunks outside its range where the chunks' transition bounds say that this is forgotten by the time its own
    // range begins (gdn_chunk_common.h, WARM_LOG2); a head with a segment that cannot is walked whole by the workgroups of segment 0.
    int nseg, seg_chunks, warm_cap;
};

// The mirror image of warm_chunks() for the scan that runs backwards: how many chunks AFTER chunk it1 - 1 a run must start from a
// zero state so that at it1 - 1 it has forgotten the difference to the true state.  When the end of the sequence comes first the
// answer is nc - it1 (the run starts from the true gradient of the final state and is exact).  -1: not within `cap` chunks.
__device__ __forceinline__ int warm_chunks_rev(const float* bound, int HV, int64_t it1, int64_t nc, int cap, int lane) {
    const bool in = lane < cap && it1 + lane < nc;
    float x = in ? bound[(it1 + lane) * HV] : 0.f;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float y = __shfl_up(x, off, 64);
        if (lane >= off) x += y;
    }
    const uint64_t hit = __builtin_amdgcn_ballot_w64(in && x <= WARM_LOG2);
    if (hit) return __builtin_ctzll(hit) + 1;
    return nc - it1 <= cap ? (int)(nc - it1) : -1;
}

// What a workgroup of the two scans does with time segments: `whole`: segment 0 walks the sequence, the others leave;
// otherwise the forward scan walks chunks [f0 - fw, f1) and keeps its results from f0 on, the reverse scan walks [f0, f1 + rw)
// downwards and keeps its results below f1.  The same in every wave of a workgroup (both scans need both answers: side by side
// in one workgroup they must take the same number of barriers).
struct ScanPlan { bool whole; int64_t f0, f1; int fw, rw; };
__device__ __forceinline__ ScanPlan scan_plan(const BwdParams& p, const SeqAt& sq, int hv, int seg, int lane) {
    ScanPlan sp{false, 0, sq.nc, 0, 0};
    if (p.nseg <= 1) return sp;
    const float* bound = p.ws.Bound + sq.cbase * p.HV + hv;
    sp.f0 = (int64_t)seg * p.seg_chunks;
    sp.f1 = seg == p.nseg - 1 ? sq.nc : (int64_t)(seg + 1) * p.seg_chunks;
    for (int s = 1; s < p.nseg; ++s) {
        const int64_t at = (int64_t)s * p.seg_chunks;           // the boundary between segments s - 1 and s
        const int fw = warm_chunks(bound, p.HV, at, p.warm_cap, lane), rw = warm_chunks_rev(bound, p.HV, at, sq.nc, p.warm_cap, lane);
        sp.whole |= fw < 0 || rw < 0;
        if (s == seg) sp.fw = fw;
        if (s == seg + 1) sp.rw = rw;
    }
    if (sp.whole) { sp.f0 = 0; sp.f1 = sq.nc; sp.fw = sp.rw = 0; }
    return sp;
}

// steps of the longer of the two scans of a workgroup
__device__ __forceinline__ int64_t pad_steps_of(const ScanPlan& sp) { return (sp.f1 - sp.f0) + (sp.fw > sp.rw ? sp.fw : sp.rw); }

// ---------------------------------------------------------------------------------------------
// prepare
// ---------------------------------------------------------------------------------------------
// (comba: a third tile of rows, those of p; the matrix L then takes the place of the q tile once q has been used, which keeps a
// workgroup at 80 KB: two per CU)
template <bool COMBA = false> constexpr size_t bwd_prep_smem() {
    return ((2 + (COMBA ? 1 : 0)) * 64 * P128 + 64 * P128 + 64 * P64) * 2 + ((COMBA ? 0 : 64 * PL) + 192) * 4;
}

// Rows of a tile on their way from memory to LDS (a row: 16 lanes next to each other, 8 features each) divided by their
// length, as gdn_l2norm_fwd does it; the normalised rows and the factors are left for the kernels that follow.
template <typename T>
__device__ __forceinline__ void l2norm_tile_rows(TileRegs<BD>& r, T* out, float* rstd_out, int H, int valid, int tid) {
    typedef typename Mma<T>::V8 V8;
    const int row0 = tid >> 4, pc = tid & 15;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        V8 x = __builtin_bit_cast(V8, r.x[i]);
        float f[8], ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { f[e] = (float)x[e]; ss += f[e] * f[e]; }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) ss += __shfl_xor(ss, off, 64);
        const float rs = rsqrtf(ss + 1e-6f);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (T)(f[e] * rs);
        r.x[i] = __builtin_bit_cast(u32x4, x);
        const int row = row0 + 16 * i;
        if (row < valid) {
            *(u32x4*)(out + (int64_t)row * H * BD + pc * 8) = r.x[i];
            if (pc == 0) rstd_out[(int64_t)row * H] = rs;
        }
    }
}

template <typename T, bool COMBA = false, bool L2 = false>
__global__ __launch_bounds__(256, 2) void gdn_bwd_prepare_kernel(BwdParams p, int64_t units) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    constexpr int KT = 1, KD = BD * KT, PK = KD + 8;             // (one block of key features; two: gdn_bwd_prepare2w_kernel)
    extern __shared__ __align__(16) char smem[];
    T* sK = (T*)smem; T* sQ = sK + 64 * PK; T* sV = sQ + 64 * PK; T* sA = sV + 64 * P128;
    T* sP = sA + 64 * P64;                                       // (comba) rows of the second key
    static_assert(!COMBA || 64 * PL * 4 <= 64 * PK * 2, "the matrix L fits the q tile");
    float* sL = COMBA ? (float*)sQ : (float*)sP;
    float* sGam = COMBA ? (float*)(sP + 64 * PK) : sL + 64 * PL; float* sBeta = sGam + 64; float* sGam0 = sBeta + 64;
    T* sRows = COMBA ? sP : sK;                                  // the rows that enter L from the left and w
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;

    // Units in turn; the next unit's rows are fetched into registers while this one is worked on.
    TileRegs<KD> rK, rQ, rP;
    TileRegs<BD> rV;
    uint32_t rG = 0, rB = 0;                                     // (raw bits: converted when the unit's turn comes)
    auto fetch = [&](int64_t u) {
        const UnitAt at = unit_at(p, u);
        const int hv = at.hv, hq = at.hq;
        const ChunkAt c = at.c;
        fetch_tile<KD>(rK, (const T*)(L2 ? p.k_raw : p.k) + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
        fetch_tile<KD>(rQ, (const T*)(L2 ? p.q_raw : p.q) + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
        if constexpr (COMBA) fetch_tile<KD>(rP, (const T*)(L2 ? p.pk_raw : p.pk) + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
        fetch_tile<BD>(rV, (const T*)p.v + (c.tok0 * p.HV + hv) * BD, (int64_t)p.HV * BD, c.valid, tid);
        rG = rB = 0;
        if (w == 0 && lane < c.valid) {
            rG = p.g ? load_scalar_bits(p.g, (c.tok0 + lane) * p.HV + hv, p.gb_dtype) : 0;
            rB = load_scalar_bits(p.beta, (c.tok0 + lane) * p.HV + hv, p.gb_dtype);
        }
    };
    fetch(blockIdx.x);
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
        // (everything derived from the lane number is derived again per unit from a copy the compiler cannot see through:
        // hoisted out of this loop, the addresses of its unrolled body would sit in registers, or spill, for its whole length)
        int tid_opaque = threadIdx.x;
        asm volatile("" : "+v"(tid_opaque));
        const int tid = tid_opaque, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
        if constexpr (L2) {
            const UnitAt at = unit_at(p, u);
            const int hv = at.hv;                      // (== the q/k head)
            const ChunkAt c = at.c;
            l2norm_tile_rows<T>(rK, (T*)p.k + (c.tok0 * p.H + hv) * KD, (float*)p.k_rstd + c.tok0 * p.H + hv, p.H, c.valid, tid);
            l2norm_tile_rows<T>(rQ, (T*)p.q + (c.tok0 * p.H + hv) * KD, (float*)p.q_rstd + c.tok0 * p.H + hv, p.H, c.valid, tid);
            if constexpr (COMBA) l2norm_tile_rows<T>(rP, (T*)p.pk + (c.tok0 * p.H + hv) * KD, (float*)p.p_rstd + c.tok0 * p.H + hv, p.H, c.valid, tid);
        }
        put_tile<KD>(sK, PK, rK, tid);
        put_tile<KD>(sQ, PK, rQ, tid);
        put_tile<BD>(sV, P128, rV, tid);
        if constexpr (COMBA) put_tile<KD>(sP, PK, rP, tid);
        if (w == 0) {
            const float g_own = scalar_of_bits(rG, p.gb_dtype);
            float x = g_own;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const float y = __shfl_up(x, off, 64);
                if (lane >= off) x += y;
            }
            sGam[lane] = x; sBeta[lane] = scalar_of_bits(rB, p.gb_dtype);
            sGam0[lane] = COMBA ? x - g_own : x;                 // (comba) the sum in front of this token: the prediction sees the state before its decay
            p.ws.Gam[u * 64 + lane] = x;
            if constexpr (COMBA) p.ws.Gam0[u * 64 + lane] = x - g_own;
        }
        lds_barrier();
        if (!COMBA && p.nseg > 1 && w == 0) {
            // how much this chunk's transition can stretch a state, in log2 units: every token's factor gamma_t (I - beta_t k_t k_t^T)
            float k2 = 0.f;
            for (int pc = 0; pc < KD / 8; ++pc) {
                const V8 kx = *(const V8*)(sK + lane * PK + pc * 8);
#pragma unroll
                for (int e = 0; e < 8; ++e) k2 += (float)kx[e] * (float)kx[e];
            }
            float lb = fabsf(1.f - sBeta[lane] * k2);
            lb = lb > 1.f ? __log2f(lb) : 0.f;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) lb += __shfl_xor(lb, off, 64);
            if (lane == 63) p.ws.Bound[u] = sGam[63] * 1.44269504f + lb;
        }
        if (u + gridDim.x < units) fetch(u + gridDim.x);

        // strip of 16 token rows per wave: L (fp32, for the substitution; entry (i, j) at [i][j % 4][j / 4]) and P^T
        {
            T* PTu = (T*)p.ws.PT + u * 64 * 64;
            f32x4 lrow[COMBA ? 4 : 1];                          // (comba) this wave's entries of L, until q's tile is free for them
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                f32x4 kk = ZERO4, qk = ZERO4;
                if (tj <= w) {
#pragma unroll
                    for (int s = 0; s < 4 * KT; ++s) {
                        const V8 b = frag_rows(sK, PK, 16 * tj, 32 * s, lane);
                        kk = Mma<T>::run(frag_rows(sRows, PK, 16 * w, 32 * s, lane), b, kk);
                        qk = Mma<T>::run(frag_rows(sQ, PK, 16 * w, 32 * s, lane), b, qk);
                    }
                }
                const int j = 16 * tj + c16;
                const float gj = sGam[j];
                f32x4 pt;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    const float d = i >= j ? __expf(sGam[i] - gj) : 0.f;
                    const float d0 = !COMBA ? d : i > j ? __expf(sGam0[i] - gj) : 0.f;
                    const float l = i > j ? sBeta[i] * kk[r] * d0 : 0.f;
                    if constexpr (COMBA) lrow[tj][r] = l;
                    else if (tj <= w) sL[i * PL + (j & 3) * 16 + (j >> 2)] = l;
                    pt[r] = p.scale * qk[r] * d;
                }
                *(V4*)(PTu + j * 64 + 16 * w + 4 * g) = pack4<T>(pt);
            }
            if constexpr (COMBA) {
                lds_barrier();                                  // (every wave has read its rows of q)
#pragma unroll
                for (int tj = 0; tj < 4; ++tj) {
                    const int j = 16 * tj + c16;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (tj <= w) sL[(16 * w + 4 * g + r) * PL + (j & 3) * 16 + (j >> 2)] = lrow[tj][r];
                }
            }
        }
        lds_barrier();
        // k -> beta e^gam k (comba: p -> beta e^gam0 p) and v -> beta v, in place
        for (int idx = tid; idx < 64 * 16 * (KT + 1); idx += 256) {
            const int row = idx / (16 * (KT + 1)), pc = idx % (16 * (KT + 1));      // the row's pieces of k, then those of v
            T* at = pc < 16 * KT ? sRows + row * PK + pc * 8 : sV + row * P128 + (pc - 16 * KT) * 8;
            const float f = pc < 16 * KT ? sBeta[row] * __expf(sGam0[row]) : sBeta[row];
            V8 x = *(V8*)at;
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * f);
            *(V8*)at = x;
        }
        solve_unit_lower_blocks<T>(sL, (float*)sA, sA, w, lane);
        lds_barrier();
        {
            T* Au = (T*)p.ws.Am + u * 64 * 64;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int idx = tid + 256 * i, row = idx >> 3, pc = idx & 7;
                *(u32x4*)(Au + row * 64 + pc * 8) = *(const u32x4*)(sA + row * P64 + pc * 8);
            }
        }
        // w^T and u^T tiles: features on the rows, this wave's 16 tokens on the columns
        {
            T* Wu = (T*)p.ws.Wm + u * 64 * KD;
            T* Uu = (T*)p.ws.Um + u * 64 * BD;
            const int i = 16 * w + c16;
            V8 fa[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) fa[s] = frag_rows(sA, P64, 16 * w, 32 * s, lane);
#pragma unroll
            for (int n = 0; n < 8 * KT; ++n) {
                f32x4 aw = ZERO4;
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (2 * s > w) continue;                    // A is lower triangular
                    aw = Mma<T>::run(frag_cols(sRows, PK, 32 * s, 16 * n, lane), fa[s], aw);
                }
                *(V4*)(Wu + i * KD + 16 * n + 4 * g) = pack4<T>(aw);
            }
#pragma unroll
            for (int n = 0; n < 8; ++n) {
                f32x4 au = ZERO4;
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (2 * s > w) continue;
                    au = Mma<T>::run(frag_cols(sV, P128, 32 * s, 16 * n, lane), fa[s], au);
                }
                *(V4*)(Uu + i * BD + 16 * n + 4 * g) = pack4<T>(au);
            }
        }
        lds_barrier();
    }
}

// Two blocks of key features in 80 KB, two workgroups per CU: k and q pass through two tile places a block of 128 features at a
// time (k k^T and q k^T add up over the blocks in registers); for w = A (beta e^gam k), which needs every block of k again, the
// second block is still in place and the first is fetched a second time, into q's place.
constexpr size_t BWD_PREP2W_SMEM = (3 * 64 * P128 + 64 * P64) * 2 + (64 * PL + 192) * 4;

template <typename T>
__global__ __launch_bounds__(256, 2) void gdn_bwd_prepare2w_kernel(BwdParams p, int64_t units) {
    static_assert(2 * BWD_PREP2W_SMEM <= 160 * 1024, "two workgroups per CU");
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    constexpr int KD = 2 * BD;
    extern __shared__ __align__(16) char smem[];
    T* sK = (T*)smem; T* sQ = sK + 64 * P128; T* sV = sQ + 64 * P128; T* sA = sV + 64 * P128;
    float* sL = (float*)(sA + 64 * P64);
    float* sGam = sL + 64 * PL; float* sBeta = sGam + 64;
    T* sK0 = sQ;                                                 // k's first block, once q is done with

    TileRegs<BD> rK, rQ, rV;
    uint32_t rG = 0, rB = 0;                                     // (raw bits: converted when the unit's turn comes)
    auto fetch_k = [&](const UnitAt& at, int kb, int tid) {
        fetch_tile<BD>(rK, (const T*)p.k + (at.c.tok0 * p.H + at.hq) * KD + BD * kb, (int64_t)p.H * KD, at.c.valid, tid);
    };
    auto fetch_q = [&](const UnitAt& at, int kb, int tid) {
        fetch_tile<BD>(rQ, (const T*)p.q + (at.c.tok0 * p.H + at.hq) * KD + BD * kb, (int64_t)p.H * KD, at.c.valid, tid);
    };
    auto fetch_rest = [&](const UnitAt& at, int tid) {           // v and the two scalars per token
        fetch_tile<BD>(rV, (const T*)p.v + (at.c.tok0 * p.HV + at.hv) * BD, (int64_t)p.HV * BD, at.c.valid, tid);
        rG = rB = 0;
        if (tid < at.c.valid) {                                  // (wave 0)
            rG = p.g ? load_scalar_bits(p.g, (at.c.tok0 + tid) * p.HV + at.hv, p.gb_dtype) : 0;
            rB = load_scalar_bits(p.beta, (at.c.tok0 + tid) * p.HV + at.hv, p.gb_dtype);
        }
    };
    {
        const UnitAt at = unit_at(p, blockIdx.x);
        fetch_k(at, 0, threadIdx.x); fetch_q(at, 0, threadIdx.x); fetch_rest(at, threadIdx.x);
    }
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
        // (everything derived from the lane number is derived again per unit from a copy the compiler cannot see through:
        // hoisted out of this loop, the addresses of its unrolled body would sit in registers, or spill, for its whole length)
        int tid_opaque = threadIdx.x;
        asm volatile("" : "+v"(tid_opaque));
        const int tid = tid_opaque, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
        const UnitAt at = unit_at(p, u);
        const bool more = u + gridDim.x < units;
        const UnitAt nx = unit_at(p, more ? u + gridDim.x : u);
        put_tile<BD>(sK, P128, rK, tid);
        put_tile<BD>(sQ, P128, rQ, tid);
        put_tile<BD>(sV, P128, rV, tid);
        if (w == 0) {
            float x = scalar_of_bits(rG, p.gb_dtype);
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const float y = __shfl_up(x, off, 64);
                if (lane >= off) x += y;
            }
            sGam[lane] = x; sBeta[lane] = scalar_of_bits(rB, p.gb_dtype);
            p.ws.Gam[u * 64 + lane] = x;
        }
        lds_barrier();
        fetch_k(at, 1, tid); fetch_q(at, 1, tid);

        // strip of 16 token rows per wave: k k^T and q k^T, a block of features at a time
        f32x4 kk[4], qk[4];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) kk[tj] = qk[tj] = ZERO4;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (kb == 1) {
                lds_barrier();                                  // (the first block is done with)
                put_tile<BD>(sK, P128, rK, tid);
                put_tile<BD>(sQ, P128, rQ, tid);
                lds_barrier();
                fetch_k(at, 0, tid);                            // (again, for w)
                if (more) { fetch_q(nx, 0, tid); fetch_rest(nx, tid); }
            }
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                if (tj <= w) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const V8 b = frag_rows(sK, P128, 16 * tj, 32 * s, lane);
                        kk[tj] = Mma<T>::run(frag_rows(sK, P128, 16 * w, 32 * s, lane), b, kk[tj]);
                        qk[tj] = Mma<T>::run(frag_rows(sQ, P128, 16 * w, 32 * s, lane), b, qk[tj]);
                    }
                }
            }
        }
        // L (fp32, for the substitution; entry (i, j) at [i][j % 4][j / 4]) and P^T
        {
            T* PTu = (T*)p.ws.PT + u * 64 * 64;
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                const int j = 16 * tj + c16;
                const float gj = sGam[j];
                f32x4 pt;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    const float d = i >= j ? __expf(sGam[i] - gj) : 0.f;
                    if (tj <= w) sL[i * PL + (j & 3) * 16 + (j >> 2)] = i > j ? sBeta[i] * kk[tj][r] * d : 0.f;
                    pt[r] = p.scale * qk[tj][r] * d;
                }
                *(V4*)(PTu + j * 64 + 16 * w + 4 * g) = pack4<T>(pt);
            }
        }
        lds_barrier();
        // k -> beta e^gam k, v -> beta v: the second block of k and v in place, the first block of k on its way into q's place
        {
            const int row0 = tid >> 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float f = sBeta[row0 + 16 * i] * __expf(sGam[row0 + 16 * i]);
                V8 x = __builtin_bit_cast(V8, rK.x[i]);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * f);
                rK.x[i] = __builtin_bit_cast(u32x4, x);
            }
            put_tile<BD>(sK0, P128, rK, tid);
            if (more) fetch_k(nx, 0, tid);
        }
        for (int idx = tid; idx < 64 * 32; idx += 256) {
            const int row = idx >> 5, pc = idx & 31;            // the row's pieces of k's second block, then those of v
            T* at2 = pc < 16 ? sK + row * P128 + pc * 8 : sV + row * P128 + (pc - 16) * 8;
            const float f = pc < 16 ? sBeta[row] * __expf(sGam[row]) : sBeta[row];
            V8 x = *(V8*)at2;
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * f);
            *(V8*)at2 = x;
        }
        solve_unit_lower_blocks<T>(sL, (float*)sA, sA, w, lane);
        lds_barrier();
        {
            T* Au = (T*)p.ws.Am + u * 64 * 64;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int idx = tid + 256 * i, row = idx >> 3, pc = idx & 7;
                *(u32x4*)(Au + row * 64 + pc * 8) = *(const u32x4*)(sA + row * P64 + pc * 8);
            }
        }
        // w^T and u^T tiles: features on the rows, this wave's 16 tokens on the columns
        {
            T* Wu = (T*)p.ws.Wm + u * 64 * KD;
            T* Uu = (T*)p.ws.Um + u * 64 * BD;
            const int i = 16 * w + c16;
            V8 fa[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) fa[s] = frag_rows(sA, P64, 16 * w, 32 * s, lane);
#pragma unroll
            for (int n = 0; n < 16; ++n) {
                const T* src = n < 8 ? sK0 : sK;
                f32x4 aw = ZERO4;
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (2 * s > w) continue;                    // A is lower triangular
                    aw = Mma<T>::run(frag_cols(src, P128, 32 * s, 16 * (n & 7), lane), fa[s], aw);
                }
                *(V4*)(Wu + i * KD + 16 * n + 4 * g) = pack4<T>(aw);
            }
#pragma unroll
            for (int n = 0; n < 8; ++n) {
                f32x4 au = ZERO4;
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (2 * s > w) continue;
                    au = Mma<T>::run(frag_cols(sV, P128, 32 * s, 16 * n, lane), fa[s], au);
                }
                *(V4*)(Uu + i * BD + 16 * n + 4 * g) = pack4<T>(au);
            }
        }
        lds_barrier();
    }
}

// ---------------------------------------------------------------------------------------------
// The two scans.  A workgroup owns VBT value columns of one (sequence, v-head): the state slice [KD][VBT] lives in
// registers as transposed tiles - wave w holds key rows KD/4 w .. as NA = KD/64 tiles (a2), lane (c16, g) key
// 16(NA w + a2) + c16 and value columns 16b + 4g .. +3.  The next chunk's tiles are fetched into registers while the
// current chunk is computed, and the barriers wait for LDS traffic only, so those loads stay in flight across them.
// ---------------------------------------------------------------------------------------------
// (the forward scan keeps v_new twice where a CU's LDS has the room: as the operand of the state update, with the decay to the end
// of the chunk on it, and as it is stored, so that it can leave as whole rows)
template <int VBT, int KT> constexpr bool state_out_tile() { return (2 * 64 * (BD * KT + 8) + BD * KT * (VBT + 8) + 2 * 64 * (VBT + 8)) * 2 + 64 * 4 <= 160 * 1024; }
template <int VBT, int KT> constexpr size_t bwd_state_smem() {
    return (2 * 64 * (BD * KT + 8) + BD * KT * (VBT + 8) + (state_out_tile<VBT, KT>() ? 2 : 1) * 64 * (VBT + 8)) * 2 + 64 * 4;
}
// (two blocks of key features at 64 columns: no room for the tile of P^T - a wave's two operand fragments of it come straight from
// memory, a step ahead like the tiles)
template <int VBT, int KT> constexpr bool dstate_pt_direct() { return KT == 2 && VBT == 64; }
template <int VBT, int KT> constexpr size_t bwd_dstate_smem() {
    return (3 * 64 * (BD * KT + 8) + (dstate_pt_direct<VBT, KT>() ? 0 : 64 * P64) + 2 * 64 * (VBT + 8) + BD * KT * (VBT + 8)) * 2 + 64 * 4;
}

// KDA: the rows of k arrive with their decay to the end of the chunk on them (KG), and the state decays per key feature (EGL).
template <typename T, int VBT, int KT, int AHEAD, int NW, bool KDA = false>
__device__ __forceinline__ void bwd_state_body(const BwdParams& p, char* smem, const int tid, const unsigned bid_all, const unsigned nwg) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    // NW waves in groups of four: a group takes VBQ of the workgroup's value columns (NB tiles per wave), every wave NA key tiles
    constexpr int PV = VBT + 8, VBQ = VBT / (NW / 4), NB = VBQ / 16, NVS = BD / VBT, KD = BD * KT, PK = KD + 8, NA = 2 * KT, NTH = 64 * NW;
    T* sW = (T*)smem; T* sK = sW + 64 * PK; T* sS = sK + 64 * PK; T* sVn = sS + KD * PV;
    constexpr bool OUT_TILE = state_out_tile<VBT, KT>();
    T* sOut = sVn + 64 * PV;                                     // v_new as it is stored (sVn: with the decay to the end of the chunk on it)
    float* sGam = (float*)(sOut + (OUT_TILE ? 64 * PV : 0));
    const int lane = tid & 63, w = (tid >> 6) & 3, vq0 = (tid >> 8) * VBQ, c16 = lane & 15, g = lane >> 4;
    // Workgroups go to the 8 XCDs in turn: the slices of one (sequence, head) take the same residue, so that they share
    // an L2 for the rows of k, q and w that all of them read.  With time segments (nwg workgroups each) a segment's come in a row.
    const int seg = p.nseg > 1 ? (int)(bid_all / (nwg / p.nseg)) : 0;
    const unsigned bid = p.nseg > 1 ? bid_all % (nwg / p.nseg) : bid_all;
    const int64_t run = (int64_t)(bid / (8 * NVS)) * 8 + bid % 8;
    if (run >= p.N * p.HV) return;
    const int vs = (bid / 8) % NVS, hv = (int)(run % p.HV), hq = hv / (p.HV / p.H);
    const int64_t n = run / p.HV;
    const SeqAt sq = seq_at(p, n);
    const int vcol0 = vs * VBT;
    const ScanPlan plan = scan_plan(p, sq, hv, seg, lane);
    if (plan.whole && seg != 0) return;
    const int64_t c_first = plan.f0 - plan.fw, c_keep = plan.f0, c_end = plan.f1;     // walks [c_first, c_end), results kept from c_keep on

    f32x4 S[NA][NB];
#pragma unroll
    for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int kk = 16 * (NA * w + a2) + c16;
            S[a2][b] = (p.h0 && c_first == 0) ? *(const f32x4*)(p.h0 + ((n * p.HV + hv) * KD + kk) * BD + vcol0 + vq0 + 16 * b + 4 * g) : ZERO4;
        }
    // (AHEAD = 2: two sets of registers take turns and the tiles of chunk c + 2 are requested while chunk c is worked on;
    // measured: no faster than one chunk of lead - a step is bound by the CU's load path, not by the way to memory)
    struct Ahead { TileRegs<KD, NTH> rW, rK; V4 rU[NB]; float rGam; float rE[NA]; };
    Ahead RA, RB;
    RA.rGam = RB.rGam = 0.f;
    auto fetch = [&](Ahead& R, int64_t ic) __attribute__((always_inline)) {
        auto& rW = R.rW; auto& rK = R.rK; auto& rU = R.rU; auto& rGam = R.rGam;
        const int64_t u = (sq.cbase + ic) * p.HV + hv, tok0 = sq.bos + ic * CH;
        const int valid = (int)min((int64_t)CH, sq.len - ic * CH);
        fetch_tile<KD, NTH>(rW, (const T*)p.ws.Wm + u * 64 * KD, KD, 64, tid);
        if constexpr (KDA) {
            fetch_tile<KD, NTH>(rK, (const T*)p.ws.KG + u * 64 * KD, KD, 64, tid);
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2) R.rE[a2] = p.ws.EGL[u * KD + 16 * (NA * w + a2) + c16];
        } else {
            fetch_tile<KD, NTH>(rK, (const T*)p.k + (tok0 * p.H + hq) * KD, (int64_t)p.H * KD, valid, tid);
            if (tid < 64) rGam = p.ws.Gam[u * 64 + tid];
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) rU[b] = *(const V4*)((const T*)p.ws.Um + u * 64 * BD + (16 * w + c16) * BD + vcol0 + vq0 + 16 * b + 4 * g);
    };
    auto step = [&](Ahead& R, int64_t ic) __attribute__((always_inline)) {
        auto& rW = R.rW; auto& rK = R.rK; auto& rU = R.rU; auto& rGam = R.rGam;
        const int64_t u = (sq.cbase + ic) * p.HV + hv;
        const bool keep = ic >= c_keep;                         // (chunks of the warm-up belong to another segment: nothing of them is stored)
        put_tile<KD, NTH>(sW, PK, rW, tid);
        put_tile<KD, NTH>(sK, PK, rK, tid);
        if (tid < 64) sGam[tid] = rGam;
        V4 u4[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) u4[b] = rU[b];
        float egk[NA];
#pragma unroll
        for (int a2 = 0; a2 < NA; ++a2) egk[a2] = R.rE[a2];
        T* Hu = (T*)p.ws.Hs + u * KD * BD;
#pragma unroll
        for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int kk = 16 * (NA * w + a2) + c16;
                *(V4*)(sS + kk * PV + vq0 + 16 * b + 4 * g) = pack4<T>(S[a2][b]);
            }
        lds_barrier();
        if (keep) copy_rows_out<KD, VBT, NTH>(Hu + vcol0, BD, sS, PV, tid);     // (whole rows of the tile: 16 bytes a lane)
        if (ic + AHEAD < c_end) fetch(R, ic + AHEAD);
        const float glast = sGam[63];
        {
            // v_new^T tiles: value columns on the rows, this wave's 16 tokens on the columns
            const int i = 16 * w + c16;
            const float dec = KDA ? 1.f : __expf(glast - sGam[i]);
            V8 wf[4 * KT];
#pragma unroll
            for (int s = 0; s < 4 * KT; ++s) wf[s] = frag_rows(sW, PK, 16 * w, 32 * s, lane);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                f32x4 acc = ZERO4;
#pragma unroll
                for (int s = 0; s < 4 * KT; ++s) acc = Mma<T>::run(frag_cols(sS, PV, 32 * s, vq0 + 16 * b, lane), wf[s], acc);
                f32x4 vn;
#pragma unroll
                for (int r = 0; r < 4; ++r) vn[r] = (float)u4[b][r] - acc[r];
                const V4 vn4 = pack4<T>(vn);
                if constexpr (OUT_TILE) *(V4*)(sOut + i * PV + vq0 + 16 * b + 4 * g) = vn4;
                else if (keep) *(V4*)((T*)p.ws.Vn + u * 64 * BD + i * BD + vcol0 + vq0 + 16 * b + 4 * g) = vn4;
#pragma unroll
                for (int r = 0; r < 4; ++r) vn[r] = (float)vn4[r] * dec;
                *(V4*)(sVn + i * PV + vq0 + 16 * b + 4 * g) = pack4<T>(vn);
            }
        }
        lds_barrier();
        if constexpr (OUT_TILE) { if (keep) copy_rows_out<64, VBT, NTH>((T*)p.ws.Vn + u * 64 * BD + vcol0, BD, sOut, PV, tid); }
        {
            const float eg = __expf(glast);
            V8 kf[NA][2];
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
                for (int s = 0; s < 2; ++s) kf[a2][s] = frag_cols(sK, PK, 32 * s, 16 * (NA * w + a2), lane);
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
                for (int b = 0; b < NB; ++b) S[a2][b] *= KDA ? egk[a2] : eg;
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const V8 fv = frag_cols(sVn, PV, 32 * s, vq0 + 16 * b, lane);
#pragma unroll
                    for (int a2 = 0; a2 < NA; ++a2) S[a2][b] = Mma<T>::run(fv, kf[a2][s], S[a2][b]);
                }
        }
        lds_barrier();
    };
    if (c_end > c_first) fetch(RA, c_first);
    if constexpr (AHEAD == 1) {
        for (int64_t ic = c_first; ic < c_end; ++ic) step(RA, ic);
    } else {
        if (c_end > c_first + 1) fetch(RB, c_first + 1);
        for (int64_t ic = c_first; ic < c_end; ic += 2) {
            step(RA, ic);
            if (ic + 1 < c_end) step(RB, ic + 1);
        }
    }
    // (side by side with the reverse scan in one workgroup: as many barriers as the longer of the two takes)
    for (int64_t i = (c_end - c_first); i < pad_steps_of(plan); ++i) { lds_barrier(); lds_barrier(); lds_barrier(); }
}

// (all 128 value columns of a head: eight waves, two per SIMD, share one set of tiles)
template <int VBT> constexpr int scan_waves() { return VBT == BD ? 8 : 4; }

template <typename T, int VBT, int KT, bool KDA = false>
__global__ __launch_bounds__(64 * scan_waves<VBT>()) void gdn_bwd_state_kernel(BwdParams p) {
    extern __shared__ __align__(16) char smem[];
    bwd_state_body<T, VBT, KT, 1, scan_waves<VBT>(), KDA>(p, smem, threadIdx.x, blockIdx.x, gridDim.x);
}

// KDA: k and q arrive as KG and QG (decays and the scale on them), P row-major instead of transposed, the gradient of the
// state decays per key feature.
template <typename T, int VBT, int KT, int AHEAD, int NW, bool KDA = false>
__device__ __forceinline__ void bwd_dstate_body(const BwdParams& p, char* smem, const int tid, const unsigned bid_all, const unsigned nwg) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    // NW waves in groups of four: a group takes VBQ of the workgroup's value columns (NB tiles per wave), every wave NA key tiles
    constexpr int PV = VBT + 8, VBQ = VBT / (NW / 4), NB = VBQ / 16, NVS = BD / VBT, KD = BD * KT, PK = KD + 8, NA = 2 * KT, NTH = 64 * NW;
    constexpr bool PT_DIRECT = dstate_pt_direct<VBT, KT>();
    static_assert(!PT_DIRECT || (!KDA && NW == 4), "fragments of P^T as the four waves of the gated delta rule read them");
    T* sK = (T*)smem; T* sQ = sK + 64 * PK; T* sW = sQ + 64 * PK; T* sPT = sW + 64 * PK;
    T* sDO = sPT + (PT_DIRECT ? 0 : 64 * P64); T* sDvn = sDO + 64 * PV; T* sDS = sDvn + 64 * PV;
    float* sGam = (float*)(sDS + KD * PV);
    const int lane = tid & 63, w = (tid >> 6) & 3, vq0 = (tid >> 8) * VBQ, c16 = lane & 15, g = lane >> 4;
    // Workgroups go to the 8 XCDs in turn: the slices of one (sequence, head) take the same residue, so that they share
    // an L2 for the rows of k, q and w that all of them read.  With time segments (nwg workgroups each) a segment's come in a row.
    const int seg = p.nseg > 1 ? (int)(bid_all / (nwg / p.nseg)) : 0;
    const unsigned bid = p.nseg > 1 ? bid_all % (nwg / p.nseg) : bid_all;
    const int64_t run = (int64_t)(bid / (8 * NVS)) * 8 + bid % 8;
    if (run >= p.N * p.HV) return;
    const int vs = (bid / 8) % NVS, hv = (int)(run % p.HV), hq = hv / (p.HV / p.H);
    const int64_t n = run / p.HV;
    const SeqAt sq = seq_at(p, n);
    const int vcol0 = vs * VBT;
    const ScanPlan plan = scan_plan(p, sq, hv, seg, lane);
    if (plan.whole && seg != 0) return;
    const int64_t c_lo = plan.f0, c_keep = plan.f1, c_top = plan.f1 + plan.rw;       // walks [c_lo, c_top) downwards, results kept below c_keep

    f32x4 dS[NA][NB];
#pragma unroll
    for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int kk = 16 * (NA * w + a2) + c16;
            dS[a2][b] = (p.dht && c_top == sq.nc) ? *(const f32x4*)(p.dht + ((n * p.HV + hv) * KD + kk) * BD + vcol0 + vq0 + 16 * b + 4 * g) : ZERO4;
        }
    // (two sets of registers for AHEAD = 2, as in the forward scan)
    // (the rows of q meet the state's gradient as scale e^gam_i q_i: a thread scales its pieces of the tile on their way into LDS, with
    // the gam of their rows fetched beside them)
    constexpr int QN = 64 * (KD / 8) / NTH, QPPR = KD / 8, QRPI = NTH / QPPR;
    struct Ahead { TileRegs<KD, NTH> rK, rQ, rW; TileRegs<CH, NTH> rPT; V8 rPf[2]; TileRegs<VBT, NTH> rDO; float rGam; float rE[NA]; float rGq[QN]; };
    Ahead RA, RB;
    RA.rGam = RB.rGam = 0.f;
    auto fetch = [&](Ahead& R, int64_t ic) __attribute__((always_inline)) {
        auto& rK = R.rK; auto& rQ = R.rQ; auto& rW = R.rW; auto& rPT = R.rPT; auto& rDO = R.rDO; auto& rGam = R.rGam;
        const int64_t u = (sq.cbase + ic) * p.HV + hv, tok0 = sq.bos + ic * CH;
        const int valid = (int)min((int64_t)CH, sq.len - ic * CH);
        if constexpr (KDA) {
            fetch_tile<KD, NTH>(rK, (const T*)p.ws.KG + u * 64 * KD, KD, 64, tid);
            fetch_tile<KD, NTH>(rQ, (const T*)p.ws.QG + u * 64 * KD, KD, 64, tid);
            fetch_tile<CH, NTH>(rPT, (const T*)p.ws.Pm + u * 64 * 64, 64, 64, tid);
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2) R.rE[a2] = p.ws.EGL[u * KD + 16 * (NA * w + a2) + c16];
        } else {
            fetch_tile<KD, NTH>(rK, (const T*)p.k + (tok0 * p.H + hq) * KD, (int64_t)p.H * KD, valid, tid);
            fetch_tile<KD, NTH>(rQ, (const T*)p.q + (tok0 * p.H + hq) * KD, (int64_t)p.H * KD, valid, tid);
            if constexpr (PT_DIRECT) {
#pragma unroll
                for (int s = 0; s < 2; ++s)
                    if (32 * s + 31 >= 16 * w) R.rPf[s] = *(const V8*)((const T*)p.ws.PT + u * 64 * 64 + (16 * w + c16) * 64 + 32 * s + 8 * g);
            } else fetch_tile<CH, NTH>(rPT, (const T*)p.ws.PT + u * 64 * 64, 64, 64, tid);
            if (tid < 64) rGam = p.ws.Gam[u * 64 + tid];
#pragma unroll
            for (int i = 0; i < QN; ++i) R.rGq[i] = p.ws.Gam[u * 64 + tid / QPPR + QRPI * i];
        }
        fetch_tile<KD, NTH>(rW, (const T*)p.ws.Wm + u * 64 * KD, KD, 64, tid);
        fetch_tile<VBT, NTH>(rDO, (const T*)p.dout + (tok0 * p.HV + hv) * BD + vcol0, (int64_t)p.HV * BD, valid, tid);
    };
    auto step = [&](Ahead& R, int64_t ic) __attribute__((always_inline)) {
        auto& rK = R.rK; auto& rQ = R.rQ; auto& rW = R.rW; auto& rPT = R.rPT; auto& rDO = R.rDO; auto& rGam = R.rGam;
        const int64_t u = (sq.cbase + ic) * p.HV + hv;
        const bool keep = ic < c_keep;                          // (chunks of the warm-up belong to another segment: nothing of them is stored)
        put_tile<KD, NTH>(sK, PK, rK, tid);
        if constexpr (!KDA) {                                   // (KDA: the factors are on the rows of q already)
#pragma unroll
            for (int i = 0; i < QN; ++i) {
                const float f = p.scale * __expf(R.rGq[i]);
                V8 x = __builtin_bit_cast(V8, rQ.x[i]);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * f);
                rQ.x[i] = __builtin_bit_cast(u32x4, x);
            }
        }
        put_tile<KD, NTH>(sQ, PK, rQ, tid);
        // (the rows of w change their sign on the way in - one bit per element - so that dv_new can stay in LDS as it is stored)
#pragma unroll
        for (int i = 0; i < (int)(sizeof(rW.x) / sizeof(rW.x[0])); ++i) rW.x[i] ^= u32x4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
        put_tile<KD, NTH>(sW, PK, rW, tid);
        if constexpr (!PT_DIRECT) put_tile<CH, NTH>(sPT, P64, rPT, tid);
        V8 pf_now[2];
        if constexpr (PT_DIRECT) { pf_now[0] = R.rPf[0]; pf_now[1] = R.rPf[1]; }
        put_tile<VBT, NTH>(sDO, PV, rDO, tid);
        if (tid < 64) sGam[tid] = rGam;
        float egk[NA];
#pragma unroll
        for (int a2 = 0; a2 < NA; ++a2) egk[a2] = R.rE[a2];
        T* dHu = (T*)p.ws.dHs + u * KD * BD;
#pragma unroll
        for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int kk = 16 * (NA * w + a2) + c16;
                *(V4*)(sDS + kk * PV + vq0 + 16 * b + 4 * g) = pack4<T>(dS[a2][b]);
            }
        lds_barrier();
        if (keep) copy_rows_out<KD, VBT, NTH>(dHu + vcol0, BD, sDS, PV, tid);
        if (ic >= c_lo + AHEAD) fetch(R, ic - AHEAD);
        const float glast = sGam[63];
        {
            // dv_new^T tiles: value columns on the rows, this wave's 16 tokens on the columns
            const int j = 16 * w + c16;
            const float dec = KDA ? 1.f : __expf(glast - sGam[j]);
            V8 kf[4 * KT], pf[2];
#pragma unroll
            for (int s = 0; s < 4 * KT; ++s) kf[s] = frag_rows(sK, PK, 16 * w, 32 * s, lane);
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                if constexpr (PT_DIRECT) pf[s] = pf_now[s];
                else pf[s] = KDA ? frag_cols(sPT, P64, 32 * s, 16 * w, lane) : frag_rows(sPT, P64, 16 * w, 32 * s, lane);
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                f32x4 a1 = ZERO4, a2v = ZERO4;
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (32 * s + 31 < 16 * w) continue;         // P^T[j][i] = 0 for i < j
                    a1 = Mma<T>::run(frag_cols(sDO, PV, 32 * s, vq0 + 16 * b, lane), pf[s], a1);
                }
#pragma unroll
                for (int s = 0; s < 4 * KT; ++s) a2v = Mma<T>::run(frag_cols(sDS, PV, 32 * s, vq0 + 16 * b, lane), kf[s], a2v);
                f32x4 dvn = a1 + a2v * dec;
                *(V4*)(sDvn + j * PV + vq0 + 16 * b + 4 * g) = pack4<T>(dvn);
            }
        }
        lds_barrier();
        if (keep) copy_rows_out<64, VBT, NTH>((T*)p.ws.dVn + u * 64 * BD + vcol0, BD, sDvn, PV, tid);
        {
            const float eg = __expf(glast);
            V8 qf[NA][2], wf[NA][2];
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    qf[a2][s] = frag_cols(sQ, PK, 32 * s, 16 * (NA * w + a2), lane);
                    wf[a2][s] = frag_cols(sW, PK, 32 * s, 16 * (NA * w + a2), lane);
                }
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
                for (int b = 0; b < NB; ++b) dS[a2][b] *= KDA ? egk[a2] : eg;
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const V8 fo = frag_cols(sDO, PV, 32 * s, vq0 + 16 * b, lane), fv = frag_cols(sDvn, PV, 32 * s, vq0 + 16 * b, lane);
#pragma unroll
                    for (int a2 = 0; a2 < NA; ++a2) {
                        dS[a2][b] = Mma<T>::run(fo, qf[a2][s], dS[a2][b]);
                        dS[a2][b] = Mma<T>::run(fv, wf[a2][s], dS[a2][b]);
                    }
                }
        }
        lds_barrier();
    };
    if (c_top > c_lo) fetch(RA, c_top - 1);
    if constexpr (AHEAD == 1) {
        for (int64_t ic = c_top - 1; ic >= c_lo; --ic) step(RA, ic);
    } else {
        if (c_top > c_lo + 1) fetch(RB, c_top - 2);
        for (int64_t ic = c_top - 1; ic >= c_lo; ic -= 2) {
            step(RA, ic);
            if (ic > c_lo) step(RB, ic - 1);
        }
    }
    for (int64_t i = (c_top - c_lo); i < pad_steps_of(plan); ++i) { lds_barrier(); lds_barrier(); lds_barrier(); }
    if (p.dh0 && c_lo == 0) {
#pragma unroll
        for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int kk = 16 * (NA * w + a2) + c16;
                *(f32x4*)(p.dh0 + ((n * p.HV + hv) * KD + kk) * BD + vcol0 + vq0 + 16 * b + 4 * g) = dS[a2][b];
            }
    }
}

template <typename T, int VBT, int KT, bool KDA = false>
__global__ __launch_bounds__(64 * scan_waves<VBT>()) void gdn_bwd_dstate_kernel(BwdParams p) {
    extern __shared__ __align__(16) char smem[];
    bwd_dstate_body<T, VBT, KT, 1, scan_waves<VBT>(), KDA>(p, smem, threadIdx.x, blockIdx.x, gridDim.x);
}

// Both scans in one workgroup of eight waves: waves 0-3 walk the chunks forwards (S, v_new), waves 4-7 backwards (dS, dv_new).
// Neither needs anything from the other and both take three barriers per chunk.  What a CU can move per step bounds both, so
// side by side they take little less than one after the other: this form serves time segments, whose workgroups already fill
// every CU (32 value columns per workgroup, one block of key features: both sets of LDS tiles fit a CU); whole sequences take
// gdn_bwd_scans_apart_kernel below.
template <int VBT, int KT> constexpr size_t bwd_scans_smem() { return bwd_state_smem<VBT, KT>() + bwd_dstate_smem<VBT, KT>(); }

template <typename T, int VBT, int KT, bool KDA = false>
__global__ __launch_bounds__(512) void gdn_bwd_scans_kernel(BwdParams p) {
    extern __shared__ __align__(16) char smem[];
    static_assert(bwd_state_smem<VBT, KT>() % 16 == 0, "the second set of tiles starts 16-byte aligned");
    if (threadIdx.x < 256) bwd_state_body<T, VBT, KT, 1, 4, KDA>(p, smem, threadIdx.x, blockIdx.x, gridDim.x);
    else bwd_dstate_body<T, VBT, KT, 1, 4, KDA>(p, smem + bwd_state_smem<VBT, KT>(), threadIdx.x - 256, blockIdx.x, gridDim.x);
}

// Both scans in one launch, in workgroups of their own: the first `nstate` workgroups walk forwards, the others backwards.
// For calls whose two scans together need no more workgroups than there are CUs: the launch then takes the time of the
// longer scan instead of their sum.
template <int VBT, int KT> constexpr size_t bwd_scans_apart_smem() {
    return bwd_state_smem<VBT, KT>() > bwd_dstate_smem<VBT, KT>() ? bwd_state_smem<VBT, KT>() : bwd_dstate_smem<VBT, KT>();
}
template <typename T, int VBT, int KT, bool KDA = false>
__global__ __launch_bounds__(64 * scan_waves<VBT>()) void gdn_bwd_scans_apart_kernel(BwdParams p, int64_t nstate) {
    extern __shared__ __align__(16) char smem[];
    if (blockIdx.x >= nstate) bwd_dstate_body<T, VBT, KT, 1, scan_waves<VBT>(), KDA>(p, smem, threadIdx.x, blockIdx.x - (unsigned)nstate, gridDim.x - (unsigned)nstate);
    else bwd_state_body<T, VBT, KT, 1, scan_waves<VBT>(), KDA>(p, smem, threadIdx.x, blockIdx.x, (unsigned)nstate);
}

// ---------------------------------------------------------------------------------------------
// dq, dw and the first parts of dk and dgam.  Per block kb of 128 key features wave w owns features 128kb + 32w .. + 31
// (two tiles a2) of all 64 tokens (four tiles t): lane (c16, g) holds token 16t + c16 and features
// 128kb + 16(2w+a2) + 4g .. +3.
// ---------------------------------------------------------------------------------------------
// One workgroup per CU walks over the units and fetches everything the next unit needs (five tiles and, with one block of key
// features, its fragments of S and dS) into registers while it works on the current one.
// L2: dq goes back through the l2 normalisation of q before it is written (its rows wait in registers for the row sums of q . dq).
template <int KT> constexpr size_t bwd_dqkw_smem() { return (3 * 64 * P128 + 2 * 64 * (BD * KT + 8) + 64 * P64) * 2 + 640 * 4; }

template <typename T, int KT, bool L2 = false>
__global__ __launch_bounds__(256, 1) void gdn_bwd_dqkw_kernel(BwdParams p, int64_t units) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    constexpr int KD = BD * KT, PK = KD + 8;
    extern __shared__ __align__(16) char smem[];
    T* sDO = (T*)smem; T* sVn = sDO + 64 * P128; T* sDvn = sVn + 64 * P128; T* sK = sDvn + 64 * P128; T* sQ = sK + 64 * PK;
    T* sDP = sQ + 64 * PK;
    float* sGam = (float*)(sDP + 64 * P64); float* sDg = sGam + 64;    // sDg [4][64]: a row per wave, added up in a fixed order (same bits every run)
    float* sQd = sDg + 256; float* sRq = sQd + 256;                    // (L2) q . dq per wave and token; the tokens' factors
    static_assert(!L2 || KT == 1, "the rows of dq wait in the registers of one block of key features");
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;

    TileRegs<BD> rDO, rVn, rDvn;
    TileRegs<KD> rK, rQ;
    V8 rS[2][4], rdS[2][4];
    float rGam = 0.f, rRq = 0.f;
    auto fetch = [&](int64_t u) {
        const UnitAt at = unit_at(p, u);
        const int hv = at.hv, hq = at.hq;
        const ChunkAt c = at.c;
        fetch_tile<BD>(rDO, (const T*)p.dout + (c.tok0 * p.HV + hv) * BD, (int64_t)p.HV * BD, c.valid, tid);
        fetch_tile<BD>(rVn, (const T*)p.ws.Vn + u * 64 * BD, BD, 64, tid);
        fetch_tile<BD>(rDvn, (const T*)p.ws.dVn + u * 64 * BD, BD, 64, tid);
        if constexpr (KT == 1) {
            const T* Hu = (const T*)p.ws.Hs + u * KD * BD;
            const T* dHu = (const T*)p.ws.dHs + u * KD * BD;
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const int kk = 16 * (2 * w + a2) + c16;
                    rS[a2][s] = *(const V8*)(Hu + kk * BD + 32 * s + 8 * g);
                    rdS[a2][s] = *(const V8*)(dHu + kk * BD + 32 * s + 8 * g);
                }
        }
        if constexpr (KT == 1) {
            fetch_tile<KD>(rK, (const T*)p.k + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
            fetch_tile<KD>(rQ, (const T*)p.q + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
        }
        if (tid < 64) rGam = p.ws.Gam[u * 64 + tid];
        if constexpr (L2) rRq = tid < c.valid ? p.q_rstd[(c.tok0 + tid) * p.H + hq] : 0.f;
    };
    fetch(blockIdx.x);
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
        const UnitAt at = unit_at(p, u);
        const int hv = at.hv;
        const ChunkAt c = at.c;
        if constexpr (KT > 1) {                                 // (no registers to spare for fetching the wide tiles ahead)
            const int hq = at.hq;
            fetch_tile<KD>(rK, (const T*)p.k + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
            fetch_tile<KD>(rQ, (const T*)p.q + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
        }
        put_tile<BD>(sDO, P128, rDO, tid);
        put_tile<BD>(sVn, P128, rVn, tid);
        put_tile<BD>(sDvn, P128, rDvn, tid);
        put_tile<KD>(sK, PK, rK, tid);
        put_tile<KD>(sQ, PK, rQ, tid);
        if (tid < 64) sGam[tid] = rGam;
        if constexpr (L2) { if (tid < 64) sRq[tid] = rRq; }
        sDg[tid] = 0.f;
        V8 sf[2][4], df[2][4];
        if constexpr (KT == 1) {
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
                for (int s = 0; s < 4; ++s) { sf[a2][s] = rS[a2][s]; df[a2][s] = rdS[a2][s]; }
        }
        lds_barrier();
        if (u + gridDim.x < units) fetch(u + gridDim.x);

        float sdot = 0.f, dglast = 0.f;
        f32x4 dq_rows[L2 ? 2 : 1][4];
#pragma unroll 1
        for (int kb = 0; kb < KT; ++kb) {                       // (a real loop: one block's accumulators at a time)
            if (KT > 1) {
                // (two blocks of key features: no registers to spare for fetching these ahead, they come straight from memory)
                const T* Hu = (const T*)p.ws.Hs + u * KD * BD;
                const T* dHu = (const T*)p.ws.dHs + u * KD * BD;
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const int kk = BD * kb + 16 * (2 * w + a2) + c16;
                        sf[a2][s] = *(const V8*)(Hu + kk * BD + 32 * s + 8 * g);
                        df[a2][s] = *(const V8*)(dHu + kk * BD + 32 * s + 8 * g);
                    }
            }
            // Operand fragments are fetched from LDS once per use across the two feature tiles of this wave.
            f32x4 G1[2][4], dKS[2][4], dWt[2][4], dPt[4];
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
                    for (int e = 0; e < 8; ++e) sdot += (float)sf[a2][s][e] * (float)df[a2][s][e];
                V8 own;
                if (kb == 0) own = frag_rows(sDO, P128, 16 * w, 32 * s, lane);      // this wave's 16 token rows of do, for dP
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
                    if (kb == 0 && t <= w) dPt[t] = Mma<T>::run(own, bvn, dPt[t]);
                }
            }
            {
                T* dWu = (T*)p.ws.dWm + u * 64 * KD;
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        *(V4*)(dWu + (16 * t + c16) * KD + BD * kb + 16 * (2 * w + a2) + 4 * g) = pack4<T>(-dWt[a2][t]);
            }
            if (kb == 0) {
                // dP o D for this wave's 16 token rows, as an operand tile
                float gi[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) gi[r] = sGam[16 * w + 4 * g + r];
#pragma unroll
                for (int tj = 0; tj < 4; ++tj) {
                    const int j = 16 * tj + c16;
                    const float gj = sGam[j];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int i = 16 * w + 4 * g + r;
                        sDP[i * P64 + j] = (T)(i >= j ? p.scale * dPt[tj][r] * __expf(gi[r] - gj) : 0.f);
                    }
                }
                lds_barrier();
            }

            const float glast = sGam[63];
            V8 fk[2][2], fq[2][2];
#pragma unroll
            for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    fk[a2][s] = frag_cols(sK, PK, 32 * s, BD * kb + 16 * (2 * w + a2), lane);
                    fq[a2][s] = frag_cols(sQ, PK, 32 * s, BD * kb + 16 * (2 * w + a2), lane);
                }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int x = 16 * t + c16;
                const float gx = sGam[x];
                const float fqs = p.scale * __expf(gx), fks = __expf(glast - gx);
                f32x4 dq[2], dk[2];
                V4 q4[2], k4[2];
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2) {
                    const int n16 = BD * kb + 16 * (2 * w + a2);
                    dq[a2] = G1[a2][t] * fqs;
                    dk[a2] = dKS[a2][t] * fks;
                    q4[a2] = *(const V4*)(sQ + x * PK + n16 + 4 * g);
                    k4[a2] = *(const V4*)(sK + x * PK + n16 + 4 * g);
#pragma unroll
                    for (int r = 0; r < 4; ++r) dglast += (float)k4[a2][r] * dk[a2][r];
                }
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (32 * s <= 16 * t + 15) {                // dP[i][j] = 0 for j > i
                        const V8 e = frag_rows(sDP, P64, 16 * t, 32 * s, lane);
#pragma unroll
                        for (int a2 = 0; a2 < 2; ++a2) dq[a2] = Mma<T>::run(fk[a2][s], e, dq[a2]);
                    }
                    if (32 * s + 31 >= 16 * t) {                // ... and for i < j
                        const V8 e = frag_cols(sDP, P64, 32 * s, 16 * t, lane);
#pragma unroll
                        for (int a2 = 0; a2 < 2; ++a2) dk[a2] = Mma<T>::run(fq[a2][s], e, dk[a2]);
                    }
                }
                float qdq = 0.f, kdk = 0.f;
#pragma unroll
                for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
                    for (int r = 0; r < 4; ++r) { qdq += (float)q4[a2][r] * dq[a2][r]; kdk += (float)k4[a2][r] * dk[a2][r]; }
                const float dgx = sum_over_g(qdq - kdk);
                if (g == 0) atomicAdd(&sDg[64 * w + x], dgx);
                if constexpr (L2) {
                    qdq = sum_over_g(qdq);
                    if (g == 0) sQd[64 * w + x] = qdq;
                    dq_rows[0][t] = dq[0]; dq_rows[1][t] = dq[1];
                }
                if (x < c.valid) {
#pragma unroll
                    for (int a2 = 0; a2 < 2; ++a2) {
                        const int n16 = BD * kb + 16 * (2 * w + a2);
                        if constexpr (!L2) *(V4*)((T*)p.dq + ((c.tok0 + x) * p.HV + hv) * KD + n16 + 4 * g) = pack4<T>(dq[a2]);
                        *(V4*)((T*)p.dk + ((c.tok0 + x) * p.HV + hv) * KD + n16 + 4 * g) = pack4<T>(dk[a2]);
                    }
                }
            }
        }
        dglast += __expf(sGam[63]) * sdot;
        dglast = sum_over_c16(sum_over_g(dglast));
        if (lane == 0) atomicAdd(&sDg[64 * w + 63], dglast);
        lds_barrier();
        if constexpr (L2) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int x = 16 * t + c16;
                const float dot = (sQd[x] + sQd[64 + x]) + (sQd[128 + x] + sQd[192 + x]), rs = sRq[x];
                if (x < c.valid) {
#pragma unroll
                    for (int a2 = 0; a2 < 2; ++a2) {
                        const int n16 = 16 * (2 * w + a2);
                        const V4 q4 = *(const V4*)(sQ + x * PK + n16 + 4 * g);
                        f32x4 out;
#pragma unroll
                        for (int r = 0; r < 4; ++r) out[r] = (dq_rows[a2][t][r] - (float)q4[r] * dot) * rs;
                        *(V4*)((T*)p.dq + ((c.tok0 + x) * p.HV + hv) * KD + n16 + 4 * g) = pack4<T>(out);
                    }
                }
            }
        }
        if (tid < 64) p.ws.Dgam[u * 64 + tid] = (sDg[tid] + sDg[64 + tid]) + (sDg[128 + tid] + sDg[192 + tid]);
        lds_barrier();
    }
}

// ---------------------------------------------------------------------------------------------
// back through w = X (e^gam k), u = X v, X = A diag(beta), A = (I + diag(beta) stril(k k^T o D))^-1
// ---------------------------------------------------------------------------------------------
// Workgroups walk over the units (chunk, v-head), the next unit's tiles on their way into registers meanwhile: dX = tril(dw (e^gam k)^T
// + du v^T), dA = stril(dX diag(beta)); dv = beta (A^T du); d(e^gam k) = beta (A^T dw), into dk, dbeta, dgam; Y = dA A^T,
// dL = -stril(A^T Y), E = diag(beta) dL o D; dk += E k + E^T k; dbeta, dgam from L = diag(beta) stril(k k^T o D); dg = the reverse
// cumulative sum of dgam inside the chunk.  sDg, sDb [4][64]: a row per wave, added up in a fixed order at the end - the same
// bits every run.
// One block of key features in at most 76 KB of LDS, so that two workgroups share a CU: the unit is walked
// in two halves over the same two tile places - first dv_new and v (dX's first term, dv and its share of dbeta), then dw and k
// (dX's second term, k k^T, the first part of dk; comba: with the rows of p in a third place) - with the second set on its way
// into registers during the first half and the next unit's first pair during the second; Y = dA A^T takes dw's place once dw is done with.
// L2: dk goes back through the l2 normalisation of k before it is written.
template <bool COMBA = false> constexpr size_t bwd_wy2_smem() { return ((2 + (COMBA ? 1 : 0)) * 64 * P128 + 2 * 64 * P64) * 2 + (960 + 640) * 4; }

template <typename T, bool L2 = false, bool COMBA = false>
__global__ __launch_bounds__(256, 2) void gdn_bwd_wy2_kernel(BwdParams p, int64_t units) {
    static_assert(2 * bwd_wy2_smem<COMBA>() <= 160 * 1024, "two workgroups per CU");
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    constexpr int KD = BD, PK = P128, NA = 2;
    extern __shared__ __align__(16) char smem[];
    T* sX0 = (T*)smem; T* sX1 = sX0 + 64 * P128;               // dv_new | v, then dw | k
    T* sA = sX1 + 64 * P128; T* sM1 = sA + 64 * P64; T* sP = sM1 + 64 * P64;     // (comba) rows of the second key
    float* sGam = (float*)(sP + (COMBA ? 64 * P128 : 0)); float* sBeta = sGam + 64; float* sDg = sBeta + 64; float* sDb = sDg + 256;
    float* sKd = sDb + 256; float* sRk = sKd + 256;              // (L2) k . dk per wave and token; the tokens' factors
    float* sDg0 = sRk + 64; float* sGam0 = sDg0 + 256;           // (comba)
    float* sPd = sGam0 + 64; float* sRp = sPd + 256;             // (comba, L2) p . dp per wave and token; the tokens' factors
    T* sDvn = sX0; T* sV = sX1; T* sDW = sX0; T* sK = sX1; T* sM2 = sX0;
    T* sRows = COMBA ? sP : sK;
    float* sGamRow = COMBA ? sGam0 : sGam; float* sDgRow = COMBA ? sDg0 : sDg;

    TileRegs<BD> rDvn, rV, rDW, rK, rP;
    TileRegs<CH> rA;
    float rGam = 0.f, rDg = 0.f, rRk = 0.f, rGam0 = 0.f, rRp = 0.f;
    uint32_t rBeta = 0;                                          // (raw bits: converted when the unit's turn comes)
    auto fetch_first = [&](int64_t u, int tid) {
        const UnitAt at = unit_at(p, u);
        const int hv = at.hv;
        const ChunkAt c = at.c;
        fetch_tile<BD>(rDvn, (const T*)p.ws.dVn + u * 64 * BD, BD, 64, tid);
        fetch_tile<BD>(rV, (const T*)p.v + (c.tok0 * p.HV + hv) * BD, (int64_t)p.HV * BD, c.valid, tid);
        fetch_tile<CH>(rA, (const T*)p.ws.Am + u * 64 * 64, 64, 64, tid);
        if (tid < 64) {
            rGam = p.ws.Gam[u * 64 + tid];
            rBeta = tid < c.valid ? load_scalar_bits(p.beta, (c.tok0 + tid) * p.HV + hv, p.gb_dtype) : 0;
            rDg = p.ws.Dgam[u * 64 + tid];
            if constexpr (COMBA) rGam0 = p.ws.Gam0[u * 64 + tid];
            if constexpr (L2) rRk = tid < c.valid ? p.k_rstd[(c.tok0 + tid) * p.H + hv] : 0.f;
            if constexpr (L2 && COMBA) rRp = tid < c.valid ? p.p_rstd[(c.tok0 + tid) * p.H + hv] : 0.f;
        }
    };
    fetch_first(blockIdx.x, threadIdx.x);
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
        // (everything derived from the lane number is derived again per unit from a copy the compiler cannot see through:
        // hoisted out of this loop, the addresses of its unrolled body would sit in registers, or spill, for its whole length)
        int tid_opaque = threadIdx.x;
        asm volatile("" : "+v"(tid_opaque));
        const int tid = tid_opaque, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
        auto feat = [&](int a) { return 16 * (2 * w + a); };    // first key feature of this wave's tile a
        const UnitAt at = unit_at(p, u);
        const int hv = at.hv, hq = at.hq;
        const ChunkAt c = at.c;
        put_tile<BD>(sDvn, P128, rDvn, tid);
        put_tile<BD>(sV, P128, rV, tid);
        put_tile<CH>(sA, P64, rA, tid);
        if (tid < 64) { sGam[tid] = rGam; sBeta[tid] = scalar_of_bits(rBeta, p.gb_dtype); if constexpr (L2) sRk[tid] = rRk; if constexpr (COMBA) sGam0[tid] = rGam0; if constexpr (L2 && COMBA) sRp[tid] = rRp; }
        sDg[tid] = tid < 64 ? rDg : 0.f;
        sDb[tid] = 0.f;
        if constexpr (COMBA) sDg0[tid] = 0.f;
        // the second pair of this unit, and what the previous kernel left in dk at this lane's places
        fetch_tile<KD>(rDW, (const T*)p.ws.dWm + u * 64 * KD, KD, 64, tid);
        fetch_tile<KD>(rK, (const T*)p.k + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
        if constexpr (COMBA) fetch_tile<KD>(rP, (const T*)p.pk + (c.tok0 * p.H + hq) * KD, (int64_t)p.H * KD, c.valid, tid);
        V4 dk_old[NA][4];
#pragma unroll
        for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int x = 16 * t + c16;
                dk_old[a2][t] = V4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
                if (x < c.valid) dk_old[a2][t] = *(const V4*)((const T*)p.dk + ((c.tok0 + x) * p.HV + hv) * KD + feat(a2) + 4 * g);
            }
        lds_barrier();

        // ---- first half: dX's first term du v^T (this wave's 16 rows i; lane: column j, rows 4g + r), and dv = beta (A^T du) ----
        f32x4 dXv[4];
        {
            V8 fa[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) fa[s] = frag_rows(sDvn, P128, 16 * w, 32 * s, lane);
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                dXv[tj] = ZERO4;
                if (tj <= w) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) dXv[tj] = Mma<T>::run(fa[s], frag_rows(sV, P128, 16 * tj, 32 * s, lane), dXv[tj]);
                }
            }
        }
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
            for (int a2 = 0; a2 < 2; ++a2) {                    // value columns 16(2w+a2) ..
                const int n16 = 16 * (2 * w + a2);
                V8 fdv[2];
#pragma unroll
                for (int s = 0; s < 2; ++s) fdv[s] = frag_cols(sDvn, P128, 32 * s, n16, lane);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    f32x4 av = ZERO4;
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        if (32 * s + 31 < 16 * t) continue;     // A[i][j] = 0 for i < j
                        av = Mma<T>::run(fdv[s], fA[t][s], av);
                    }
                    const int j = 16 * t + c16;
                    const V4 v4 = *(const V4*)(sV + j * P128 + n16 + 4 * g);
                    float dbv = 0.f;
#pragma unroll
                    for (int r = 0; r < 4; ++r) dbv += av[r] * (float)v4[r];
                    dbv = sum_over_g(dbv);
                    if (g == 0) atomicAdd(&sDb[64 * w + j], dbv);
                    if (j < c.valid) *(V4*)((T*)p.dv + ((c.tok0 + j) * p.HV + hv) * BD + n16 + 4 * g) = pack4<T>(av * bj[t]);
                }
            }
        }
        lds_barrier();                                          // (dv_new and v are done with)
        put_tile<KD>(sDW, PK, rDW, tid);
        put_tile<KD>(sK, PK, rK, tid);
        if constexpr (COMBA) put_tile<KD>(sP, PK, rP, tid);
        lds_barrier();
        if (u + gridDim.x < units) fetch_first(u + gridDim.x, tid);

        // ---- second half: dX's second term dw (e^gam k)^T, dA = stril(dX diag(beta)), k k^T of the same rows and columns ----
        // (comba: e^gam0 p in k's place wherever k stood on the left of k k^T or under e^gam)
        f32x4 kkT[4];
        {
            V8 fw[4], fk[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                fw[s] = frag_rows(sDW, PK, 16 * w, 32 * s, lane);
                fk[s] = frag_rows(sRows, PK, 16 * w, 32 * s, lane);
            }
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                f32x4 dXw = ZERO4;
                kkT[tj] = ZERO4;
                if (tj <= w) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const V8 bk = frag_rows(sK, PK, 16 * tj, 32 * s, lane);
                        if constexpr (COMBA) dXw = Mma<T>::run(fw[s], frag_rows(sP, PK, 16 * tj, 32 * s, lane), dXw);
                        else dXw = Mma<T>::run(fw[s], bk, dXw);
                        kkT[tj] = Mma<T>::run(fk[s], bk, kkT[tj]);
                    }
                }
                const int j = 16 * tj + c16;
                const float ej = __expf(sGamRow[j]), bj = sBeta[j];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    sM1[i * P64 + j] = (T)(i > j ? (dXv[tj][r] + ej * dXw[r]) * bj : 0.f);
                }
            }
        }
        // d(e^gam k) = beta (A^T dw): into dk, dbeta, dgam  (comba: d(e^gam0 p), into dp, dbeta, dgam0)
        f32x4 dk[NA][4], dpk[COMBA ? NA : 1][4];
        {
            V8 fA[4][2];
            float ej[4], bj[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int s = 0; s < 2; ++s)
                    if (32 * s + 31 >= 16 * t) fA[t][s] = frag_cols(sA, P64, 32 * s, 16 * t, lane);
                ej[t] = __expf(sGamRow[16 * t + c16]);
                bj[t] = sBeta[16 * t + c16];
            }
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2) {                   // key features feat(a2) ..
                const int n16 = feat(a2);
                V8 fdw[2];
#pragma unroll
                for (int s = 0; s < 2; ++s) fdw[s] = frag_cols(sDW, PK, 32 * s, n16, lane);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    f32x4 ak = ZERO4;
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        if (32 * s + 31 < 16 * t) continue;
                        ak = Mma<T>::run(fdw[s], fA[t][s], ak);
                    }
                    const int j = 16 * t + c16;
                    const V4 k4 = *(const V4*)(sRows + j * PK + n16 + 4 * g);
                    float dot = 0.f;
#pragma unroll
                    for (int r = 0; r < 4; ++r) dot += ak[r] * (float)k4[r];
                    dot = sum_over_g(dot);
                    if (g == 0) { atomicAdd(&sDb[64 * w + j], ej[t] * dot); atomicAdd(&sDgRow[64 * w + j], bj[t] * ej[t] * dot); }
                    if constexpr (COMBA) { dpk[a2][t] = ak * (bj[t] * ej[t]); dk[a2][t] = ZERO4; }
                    else dk[a2][t] = ak * (bj[t] * ej[t]);
                }
            }
        }
        lds_barrier();
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
        // dL = -stril(A^T Y);  E = diag(beta) dL o D as an operand tile;  dbeta, dgam from L = diag(beta) stril(k k^T o D)
        {
            float dbi[4] = {0.f, 0.f, 0.f, 0.f}, rowF[4] = {0.f, 0.f, 0.f, 0.f}, gi[4], bi[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) { gi[r] = sGamRow[16 * w + 4 * g + r]; bi[r] = sBeta[16 * w + 4 * g + r]; }
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
                const f32x4 kk = kkT[tl];
                const int l = 16 * tl + c16;
                const float gl = sGam[l];
                float colF = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    float E = 0.f;
                    if (i > l) {
                        const float d = __expf(gi[r] - gl), dL = -acc[r];
                        dbi[r] += dL * kk[r] * d;
                        E = dL * bi[r] * d;
                        const float F = E * kk[r];
                        rowF[r] += F;
                        colF += F;
                    }
                    sM1[i * P64 + l] = (T)E;
                }
                colF = sum_over_g(colF);
                if (g == 0 && tl <= w) atomicAdd(&sDg[64 * w + l], -colF);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float a = sum_over_c16(dbi[r]), b = sum_over_c16(rowF[r]);
                if (c16 == 0) { atomicAdd(&sDb[64 * w + 16 * w + 4 * g + r], a); atomicAdd(&sDgRow[64 * w + 16 * w + 4 * g + r], b); }
            }
        }
        lds_barrier();
        // dk += E k + E^T k, on top of what the previous kernel left  (comba: dp += E k, dk += E^T p)
        {
            V8 fk[NA][2], fp[COMBA ? NA : 1][2];
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    fk[a2][s] = frag_cols(sK, PK, 32 * s, feat(a2), lane);
                    if constexpr (COMBA) fp[a2][s] = frag_cols(sP, PK, 32 * s, feat(a2), lane);
                }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (32 * s <= 16 * t + 15) {                // E[i][l], l < i
                        const V8 e = frag_rows(sM1, P64, 16 * t, 32 * s, lane);
#pragma unroll
                        for (int a2 = 0; a2 < NA; ++a2) {
                            if constexpr (COMBA) dpk[a2][t] = Mma<T>::run(fk[a2][s], e, dpk[a2][t]);
                            else dk[a2][t] = Mma<T>::run(fk[a2][s], e, dk[a2][t]);
                        }
                    }
                    if (32 * s + 31 >= 16 * t) {                // E[i][l], i > l
                        const V8 e = frag_cols(sM1, P64, 32 * s, 16 * t, lane);
#pragma unroll
                        for (int a2 = 0; a2 < NA; ++a2) {
                            if constexpr (COMBA) dk[a2][t] = Mma<T>::run(fp[a2][s], e, dk[a2][t]);
                            else dk[a2][t] = Mma<T>::run(fk[a2][s], e, dk[a2][t]);
                        }
                    }
                }
                const int x = 16 * t + c16;
                if constexpr (L2) {
                    float kdk = 0.f;
#pragma unroll
                    for (int a2 = 0; a2 < NA; ++a2) {
                        const V4 k4 = *(const V4*)(sK + x * PK + feat(a2) + 4 * g);
#pragma unroll
                        for (int r = 0; r < 4; ++r) { dk[a2][t][r] += (float)dk_old[a2][t][r]; kdk += (float)k4[r] * dk[a2][t][r]; }
                    }
                    kdk = sum_over_g(kdk);
                    if (g == 0) sKd[64 * w + x] = kdk;
                    if constexpr (COMBA) {
                        float pdp = 0.f;
#pragma unroll
                        for (int a2 = 0; a2 < NA; ++a2) {
                            const V4 p4 = *(const V4*)(sP + x * PK + feat(a2) + 4 * g);
#pragma unroll
                            for (int r = 0; r < 4; ++r) pdp += (float)p4[r] * dpk[a2][t][r];
                        }
                        pdp = sum_over_g(pdp);
                        if (g == 0) sPd[64 * w + x] = pdp;
                    }
                } else if (x < c.valid) {
#pragma unroll
                    for (int a2 = 0; a2 < NA; ++a2) {
                        f32x4 acc = dk[a2][t];
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[r] += (float)dk_old[a2][t][r];
                        *(V4*)((T*)p.dk + ((c.tok0 + x) * p.HV + hv) * KD + feat(a2) + 4 * g) = pack4<T>(acc);
                        if constexpr (COMBA) *(V4*)((T*)p.dp + ((c.tok0 + x) * p.HV + hv) * KD + feat(a2) + 4 * g) = pack4<T>(dpk[a2][t]);
                    }
                }
            }
        }
        if constexpr (L2) {
            lds_barrier();
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int x = 16 * t + c16;
                const float dot = (sKd[x] + sKd[64 + x]) + (sKd[128 + x] + sKd[192 + x]), rs = sRk[x];
                if (x < c.valid) {
#pragma unroll
                    for (int a2 = 0; a2 < NA; ++a2) {
                        const V4 k4 = *(const V4*)(sK + x * PK + feat(a2) + 4 * g);
                        f32x4 out;
#pragma unroll
                        for (int r = 0; r < 4; ++r) out[r] = (dk[a2][t][r] - (float)k4[r] * dot) * rs;
                        *(V4*)((T*)p.dk + ((c.tok0 + x) * p.HV + hv) * KD + feat(a2) + 4 * g) = pack4<T>(out);
                    }
                }
                if constexpr (COMBA) {
                    const float dotp = (sPd[x] + sPd[64 + x]) + (sPd[128 + x] + sPd[192 + x]), rp = sRp[x];
                    if (x < c.valid) {
#pragma unroll
                        for (int a2 = 0; a2 < NA; ++a2) {
                            const V4 p4 = *(const V4*)(sP + x * PK + feat(a2) + 4 * g);
                            f32x4 out;
#pragma unroll
                            for (int r = 0; r < 4; ++r) out[r] = (dpk[a2][t][r] - (float)p4[r] * dotp) * rp;
                            *(V4*)((T*)p.dp + ((c.tok0 + x) * p.HV + hv) * KD + feat(a2) + 4 * g) = pack4<T>(out);
                        }
                    }
                }
            }
        }
        if (w == 0) {
            float x = (sDg[lane] + sDg[64 + lane]) + (sDg[128 + lane] + sDg[192 + lane]);
            // (comba) dg_t = sum_{s >= t} dgam_s + sum_{s > t} dgam0_s: one reverse cumulative sum of both, less the token's own dgam0
            float own0 = 0.f;
            if constexpr (COMBA) { own0 = (sDg0[lane] + sDg0[64 + lane]) + (sDg0[128 + lane] + sDg0[192 + lane]); x += own0; }
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const float y = __shfl_down(x, off, 64);
                if (lane + off < 64) x += y;
            }
            x -= own0;
            if (lane < c.valid) {
                p.dg[(c.tok0 + lane) * p.HV + hv] = x;
                p.dbeta[(c.tok0 + lane) * p.HV + hv] = (sDb[lane] + sDb[64 + lane]) + (sDb[128 + lane] + sDb[192 + lane]);
            }
        }
        lds_barrier();
    }
}

// The same in two halves for two blocks of key features, still two workgroups per CU: the second half takes dw and k one block of
// 128 features at a time through the same two tile places (the products with dw and k add up over the blocks; d(e^gam k) of a
// block needs that block only), and the last step goes over the blocks again, k's first block fetched a second time.
constexpr size_t BWD_WY2W_SMEM = (2 * 64 * P128 + 2 * 64 * P64) * 2 + 640 * 4;

template <typename T>
__global__ __launch_bounds__(256, 2) void gdn_bwd_wy2w_kernel(BwdParams p, int64_t units) {
    static_assert(2 * BWD_WY2W_SMEM <= 160 * 1024, "two workgroups per CU");
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    constexpr int KD = 2 * BD, PK = P128, NA = 2;
    extern __shared__ __align__(16) char smem[];
    T* sX0 = (T*)smem; T* sX1 = sX0 + 64 * P128;               // dv_new | v, then a block of dw | k
    T* sA = sX1 + 64 * P128; T* sM1 = sA + 64 * P64;
    float* sGam = (float*)(sM1 + 64 * P64); float* sBeta = sGam + 64; float* sDg = sBeta + 64; float* sDb = sDg + 256;
    T* sDvn = sX0; T* sV = sX1; T* sDW = sX0; T* sK = sX1; T* sM2 = sX0;

    TileRegs<BD> rDvn, rV, rDW, rK;
    TileRegs<CH> rA;
    float rGam = 0.f, rDg = 0.f;
    uint32_t rBeta = 0;                                          // (raw bits: converted when the unit's turn comes)
    auto fetch_first = [&](int64_t u, int tid) {
        const UnitAt at = unit_at(p, u);
        const ChunkAt c = at.c;
        fetch_tile<BD>(rDvn, (const T*)p.ws.dVn + u * 64 * BD, BD, 64, tid);
        fetch_tile<BD>(rV, (const T*)p.v + (c.tok0 * p.HV + at.hv) * BD, (int64_t)p.HV * BD, c.valid, tid);
        fetch_tile<CH>(rA, (const T*)p.ws.Am + u * 64 * 64, 64, 64, tid);
        if (tid < 64) {
            rGam = p.ws.Gam[u * 64 + tid];
            rBeta = tid < c.valid ? load_scalar_bits(p.beta, (c.tok0 + tid) * p.HV + at.hv, p.gb_dtype) : 0;
            rDg = p.ws.Dgam[u * 64 + tid];
        }
    };
    fetch_first(blockIdx.x, threadIdx.x);
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
        // (everything derived from the lane number is derived again per unit from a copy the compiler cannot see through:
        // hoisted out of this loop, the addresses of its unrolled body would sit in registers, or spill, for its whole length)
        int tid_opaque = threadIdx.x;
        asm volatile("" : "+v"(tid_opaque));
        const int tid = tid_opaque, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c16 = lane & 15, g = lane >> 4;
        auto feat = [&](int a) { return 16 * (2 * w + a); };    // first key feature, inside a block, of this wave's tile a
        const UnitAt at = unit_at(p, u);
        const int hv = at.hv, hq = at.hq;
        const ChunkAt c = at.c;
        auto fetch_dw = [&](int kb) { fetch_tile<BD>(rDW, (const T*)p.ws.dWm + u * 64 * KD + BD * kb, KD, 64, tid); };
        auto fetch_k = [&](int kb) { fetch_tile<BD>(rK, (const T*)p.k + (c.tok0 * p.H + hq) * KD + BD * kb, (int64_t)p.H * KD, c.valid, tid); };
        put_tile<BD>(sDvn, P128, rDvn, tid);
        put_tile<BD>(sV, P128, rV, tid);
        put_tile<CH>(sA, P64, rA, tid);
        if (tid < 64) { sGam[tid] = rGam; sBeta[tid] = scalar_of_bits(rBeta, p.gb_dtype); }
        sDg[tid] = tid < 64 ? rDg : 0.f;
        sDb[tid] = 0.f;
        fetch_dw(0);
        fetch_k(0);
        lds_barrier();

        // ---- first half: dX's first term du v^T (this wave's 16 rows i; lane: column j, rows 4g + r), and dv = beta (A^T du) ----
        f32x4 dXv[4];
        {
            V8 fa[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) fa[s] = frag_rows(sDvn, P128, 16 * w, 32 * s, lane);
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) {
                dXv[tj] = ZERO4;
                if (tj <= w) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) dXv[tj] = Mma<T>::run(fa[s], frag_rows(sV, P128, 16 * tj, 32 * s, lane), dXv[tj]);
                }
            }
        }
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
            for (int a2 = 0; a2 < 2; ++a2) {                    // value columns 16(2w+a2) ..
                const int n16 = 16 * (2 * w + a2);
                V8 fdv[2];
#pragma unroll
                for (int s = 0; s < 2; ++s) fdv[s] = frag_cols(sDvn, P128, 32 * s, n16, lane);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    f32x4 av = ZERO4;
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        if (32 * s + 31 < 16 * t) continue;     // A[i][j] = 0 for i < j
                        av = Mma<T>::run(fdv[s], fA[t][s], av);
                    }
                    const int j = 16 * t + c16;
                    const V4 v4 = *(const V4*)(sV + j * P128 + n16 + 4 * g);
                    float dbv = 0.f;
#pragma unroll
                    for (int r = 0; r < 4; ++r) dbv += av[r] * (float)v4[r];
                    dbv = sum_over_g(dbv);
                    if (g == 0) atomicAdd(&sDb[64 * w + j], dbv);
                    if (j < c.valid) *(V4*)((T*)p.dv + ((c.tok0 + j) * p.HV + hv) * BD + n16 + 4 * g) = pack4<T>(av * bj[t]);
                }
            }
        }

        // ---- second half, a block of key features at a time: dX's second term dw (e^gam k)^T and k k^T add up over the blocks;
        // d(e^gam k) = beta (A^T dw) of a block goes into that block's dk, and into dbeta, dgam ----
        f32x4 dXw[4], kkT[4], dk[2][NA][4];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) dXw[tj] = kkT[tj] = ZERO4;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            lds_barrier();                                      // (the two tile places are done with)
            put_tile<BD>(sDW, PK, rDW, tid);
            put_tile<BD>(sK, PK, rK, tid);
            lds_barrier();
            if (kb == 0) { fetch_dw(1); fetch_k(1); }
            else {
                if (u + gridDim.x < units) fetch_first(u + gridDim.x, tid);
                fetch_k(0);                                     // (for the last step)
            }
            {
                V8 fw[4], fk[4];
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    fw[s] = frag_rows(sDW, PK, 16 * w, 32 * s, lane);
                    fk[s] = frag_rows(sK, PK, 16 * w, 32 * s, lane);
                }
#pragma unroll
                for (int tj = 0; tj < 4; ++tj) {
                    if (tj <= w) {
#pragma unroll
                        for (int s = 0; s < 4; ++s) {
                            const V8 bk = frag_rows(sK, PK, 16 * tj, 32 * s, lane);
                            dXw[tj] = Mma<T>::run(fw[s], bk, dXw[tj]);
                            kkT[tj] = Mma<T>::run(fk[s], bk, kkT[tj]);
                        }
                    }
                }
            }
            {
                V8 fA[4][2];
                float ej[4], bj[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
#pragma unroll
                    for (int s = 0; s < 2; ++s)
                        if (32 * s + 31 >= 16 * t) fA[t][s] = frag_cols(sA, P64, 32 * s, 16 * t, lane);
                    ej[t] = __expf(sGam[16 * t + c16]);
                    bj[t] = sBeta[16 * t + c16];
                }
#pragma unroll
                for (int a2 = 0; a2 < NA; ++a2) {               // key features 128 kb + feat(a2) ..
                    const int n16 = feat(a2);
                    V8 fdw[2];
#pragma unroll
                    for (int s = 0; s < 2; ++s) fdw[s] = frag_cols(sDW, PK, 32 * s, n16, lane);
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        f32x4 ak = ZERO4;
#pragma unroll
                        for (int s = 0; s < 2; ++s) {
                            if (32 * s + 31 < 16 * t) continue;
                            ak = Mma<T>::run(fdw[s], fA[t][s], ak);
                        }
                        const int j = 16 * t + c16;
                        const V4 k4 = *(const V4*)(sK + j * PK + n16 + 4 * g);
                        float dot = 0.f;
#pragma unroll
                        for (int r = 0; r < 4; ++r) dot += ak[r] * (float)k4[r];
                        dot = sum_over_g(dot);
                        if (g == 0) { atomicAdd(&sDb[64 * w + j], ej[t] * dot); atomicAdd(&sDg[64 * w + j], bj[t] * ej[t] * dot); }
                        dk[kb][a2][t] = ak * (bj[t] * ej[t]);
                    }
                }
            }
        }
        // dA = stril(dX diag(beta))
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            const int j = 16 * tj + c16;
            const float ej = __expf(sGam[j]), bj = sBeta[j];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 16 * w + 4 * g + r;
                sM1[i * P64 + j] = (T)(i > j ? (dXv[tj][r] + ej * dXw[tj][r]) * bj : 0.f);
            }
        }
        lds_barrier();
        // Y = dA A^T  (into dw's place)
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
        // dL = -stril(A^T Y);  E = diag(beta) dL o D as an operand tile;  dbeta, dgam from L = diag(beta) stril(k k^T o D)
        {
            float dbi[4] = {0.f, 0.f, 0.f, 0.f}, rowF[4] = {0.f, 0.f, 0.f, 0.f}, gi[4], bi[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) { gi[r] = sGam[16 * w + 4 * g + r]; bi[r] = sBeta[16 * w + 4 * g + r]; }
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
                const f32x4 kk = kkT[tl];
                const int l = 16 * tl + c16;
                const float gl = sGam[l];
                float colF = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int i = 16 * w + 4 * g + r;
                    float E = 0.f;
                    if (i > l) {
                        const float d = __expf(gi[r] - gl), dL = -acc[r];
                        dbi[r] += dL * kk[r] * d;
                        E = dL * bi[r] * d;
                        const float F = E * kk[r];
                        rowF[r] += F;
                        colF += F;
                    }
                    sM1[i * P64 + l] = (T)E;
                }
                colF = sum_over_g(colF);
                if (g == 0 && tl <= w) atomicAdd(&sDg[64 * w + l], -colF);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float a = sum_over_c16(dbi[r]), b = sum_over_c16(rowF[r]);
                if (c16 == 0) { atomicAdd(&sDb[64 * w + 16 * w + 4 * g + r], a); atomicAdd(&sDg[64 * w + 16 * w + 4 * g + r], b); }
            }
        }
        // dk += E k + E^T k, on top of what the previous kernel left: the second block (its rows of k are in place), then the first
#pragma unroll
        for (int kb = 1; kb >= 0; --kb) {
            V4 dk_old[NA][4];
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int x = 16 * t + c16;
                    dk_old[a2][t] = V4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
                    if (x < c.valid) dk_old[a2][t] = *(const V4*)((const T*)p.dk + ((c.tok0 + x) * p.HV + hv) * KD + BD * kb + feat(a2) + 4 * g);
                }
            lds_barrier();                                      // (E is complete; second round: the second block's rows are done with)
            if (kb == 0) {
                put_tile<BD>(sK, PK, rK, tid);
                lds_barrier();
            }
            V8 fk[NA][2];
#pragma unroll
            for (int a2 = 0; a2 < NA; ++a2)
#pragma unroll
                for (int s = 0; s < 2; ++s) fk[a2][s] = frag_cols(sK, PK, 32 * s, feat(a2), lane);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    if (32 * s <= 16 * t + 15) {                // E[i][l], l < i
                        const V8 e = frag_rows(sM1, P64, 16 * t, 32 * s, lane);
#pragma unroll
                        for (int a2 = 0; a2 < NA; ++a2) dk[kb][a2][t] = Mma<T>::run(fk[a2][s], e, dk[kb][a2][t]);
                    }
                    if (32 * s + 31 >= 16 * t) {                // E[i][l], i > l
                        const V8 e = frag_cols(sM1, P64, 32 * s, 16 * t, lane);
#pragma unroll
                        for (int a2 = 0; a2 < NA; ++a2) dk[kb][a2][t] = Mma<T>::run(fk[a2][s], e, dk[kb][a2][t]);
                    }
                }
                const int x = 16 * t + c16;
                if (x < c.valid) {
#pragma unroll
                    for (int a2 = 0; a2 < NA; ++a2) {
                        f32x4 acc = dk[kb][a2][t];
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[r] += (float)dk_old[a2][t][r];
                        *(V4*)((T*)p.dk + ((c.tok0 + x) * p.HV + hv) * KD + BD * kb + feat(a2) + 4 * g) = pack4<T>(acc);
                    }
                }
            }
        }
        if (w == 0) {
            float x = (sDg[lane] + sDg[64 + lane]) + (sDg[128 + lane] + sDg[192 + lane]);
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const float y = __shfl_down(x, off, 64);
                if (lane + off < 64) x += y;
            }
            if (lane < c.valid) {
                p.dg[(c.tok0 + lane) * p.HV + hv] = x;
                p.dbeta[(c.tok0 + lane) * p.HV + hv] = (sDb[lane] + sDb[64 + lane]) + (sDb[128 + lane] + sDb[192 + lane]);
            }
        }
        lds_barrier();
    }
}

template <typename T, int KT, bool COMBA = false>
static int launch_bwd(const BwdParams& p_in, int64_t num_chunks, hipStream_t stream) {
    BwdParams p = p_in;
    // Value columns per workgroup of the scans where the two run one after the other or side by side in one workgroup: as few as
    // it takes to give every (sequence, head) run its own CU (their LDS tiles allow one workgroup per CU).  With two blocks of
    // key features the reverse scan's tiles leave room for 64 columns at most (taken where 64-column slices fill the chip: each
    // slice reads the head's rows of k, q and w again, 96 KB a step).
    const int64_t runs1 = p.N * p.HV;
    const int vbt = runs1 <= 64 ? 32 : runs1 <= 128 ? 64 : 128;
    const int vbt_d = KT == 1 ? vbt : runs1 >= 128 ? 64 : 32;
    const unsigned units = (unsigned)(num_chunks * p.HV);
    auto runs = [&](int v) { return (unsigned)((runs1 + 7) / 8 * 8 * (BD / v)); };
    struct K { const void* f; size_t smem; const char* name; unsigned grid; };
    K state, dstate;
    if (vbt == 32) state = {(const void*)gdn_bwd_state_kernel<T, 32, KT>, bwd_state_smem<32, KT>(), "gdn_bwd_state_kernel", runs(32)};
    else if (vbt == 64) state = {(const void*)gdn_bwd_state_kernel<T, 64, KT>, bwd_state_smem<64, KT>(), "gdn_bwd_state_kernel", runs(64)};
    else state = {(const void*)gdn_bwd_state_kernel<T, 128, KT>, bwd_state_smem<128, KT>(), "gdn_bwd_state_kernel", runs(128)};
    if (vbt_d == 32) dstate = {(const void*)gdn_bwd_dstate_kernel<T, 32, KT>, bwd_dstate_smem<32, KT>(), "gdn_bwd_dstate_kernel", runs(32)};
    else if (vbt_d == 64) dstate = {(const void*)gdn_bwd_dstate_kernel<T, 64, KT>, bwd_dstate_smem<64, KT>(), "gdn_bwd_dstate_kernel", runs(64)};
    else if constexpr (KT == 1) dstate = {(const void*)gdn_bwd_dstate_kernel<T, 128, KT>, bwd_dstate_smem<128, KT>(), "gdn_bwd_dstate_kernel", runs(128)};
    unsigned threads[5] = {256, vbt == BD ? 512u : 256u, vbt_d == BD ? 512u : 256u, 256, 256};
    if constexpr (KT == 1) {
        // both scans side by side in one launch (the second entry then has nothing to launch): what time segments run in, where
        // every CU has a workgroup already
        if (vbt == 32) {
            state = {(const void*)gdn_bwd_scans_kernel<T, 32, KT>, bwd_scans_smem<32, KT>(), "gdn_bwd_scans_kernel", runs(32)};
            threads[1] = 512;
            dstate.grid = 0;
        }
    }
    // Time segments for the two scans (one block of key features, dense input): long sequences on few heads leave CUs without a
    // workgroup; never more workgroups than CUs, segments of 8 chunks or more, and at least 24 steps saved per workgroup
    // (a warm-up of typical length must pay).  GDN_FLAG_SCAN_WIDE asks for whole sequences, GDN_FLAG_SCAN_SEGMENTS for segments of 4.
    p.nseg = 1; p.seg_chunks = (int)p.NT; p.warm_cap = 0;
    if constexpr (KT == 1 && !COMBA) {
        if (!p.cu_seqlens && vbt == 32 && !(p.flags & GDN_FLAG_SCAN_WIDE)) {
            const bool force = p.flags & GDN_FLAG_SCAN_SEGMENTS;
            int nseg = (int)std::min<int64_t>(256 / runs(32), p.NT / (force ? 4 : 8));
            if (nseg >= 2 && (force || p.NT - p.NT / nseg >= 24)) {
                p.nseg = nseg;
                p.seg_chunks = (int)((p.NT + nseg - 1) / nseg);
                p.warm_cap = std::min(WARM_CAP_MAX, p.seg_chunks + p.seg_chunks / 4 + 6);
                state.grid *= nseg;                             // (vbt = 32: the two scans side by side)
            }
        }
    }
    int64_t second_arg[5] = {units, units, units, units, units};    // (the kernels that walk over the units take their number)
    if (vbt == 32 && vbt_d == 32 && dstate.grid != 0 && state.grid + dstate.grid <= 256u) {
        // both scans in one launch, each in workgroups of its own (the second entry then has nothing to launch)
        second_arg[1] = state.grid;
        state = {(const void*)gdn_bwd_scans_apart_kernel<T, 32, KT>, bwd_scans_apart_smem<32, KT>(), "gdn_bwd_scans_apart_kernel", state.grid + dstate.grid};
        dstate.grid = 0;
    }
    if constexpr (KT == 1) {
        // Whole sequences on up to 128 runs: both scans in one launch, every workgroup with a CU to itself, as many value columns
        // each as that allows.  What a CU moves per step bounds the step (some 22 GB/s per CU, loads and stores together, whatever
        // shares the CU): 32 KB + c/2 for c columns of the forward scan, 56 KB + c/2 of the reverse one - side by side in one
        // workgroup the two add up, apart the longer one counts.
        if (p.nseg == 1 && runs1 <= 128) {
            const int va = runs1 <= 32 ? 32 : runs1 <= 64 ? 64 : 128;
            second_arg[1] = runs(va);
            threads[1] = va == BD ? 512u : 256u;
            if (va == 32) state = {(const void*)gdn_bwd_scans_apart_kernel<T, 32, KT>, bwd_scans_apart_smem<32, KT>(), "gdn_bwd_scans_apart_kernel", 2 * runs(32)};
            else if (va == 64) state = {(const void*)gdn_bwd_scans_apart_kernel<T, 64, KT>, bwd_scans_apart_smem<64, KT>(), "gdn_bwd_scans_apart_kernel", 2 * runs(64)};
            else state = {(const void*)gdn_bwd_scans_apart_kernel<T, 128, KT>, bwd_scans_apart_smem<128, KT>(), "gdn_bwd_scans_apart_kernel", 2 * runs(128)};
            dstate.grid = 0;
        }
    }
    const bool l2 = KT == 1 && p.q_raw;                     // (the entry has checked H == HV)
    K prep;
    if constexpr (KT == 1) prep = {l2 ? (const void*)gdn_bwd_prepare_kernel<T, COMBA, true> : (const void*)gdn_bwd_prepare_kernel<T, COMBA>, bwd_prep_smem<COMBA>(), "gdn_bwd_prepare_kernel", units < 512u ? units : 512u};
    else prep = {(const void*)gdn_bwd_prepare2w_kernel<T>, BWD_PREP2W_SMEM, "gdn_bwd_prepare2w_kernel", units < 512u ? units : 512u};
    K wy;
    if constexpr (KT == 1) wy = {l2 ? (const void*)gdn_bwd_wy2_kernel<T, true, COMBA> : (const void*)gdn_bwd_wy2_kernel<T, false, COMBA>, bwd_wy2_smem<COMBA>(), "gdn_bwd_wy2_kernel", units < 512u ? units : 512u};
    else wy = {(const void*)gdn_bwd_wy2w_kernel<T>, BWD_WY2W_SMEM, "gdn_bwd_wy2w_kernel", units < 512u ? units : 512u};
    const K ks[5] = {
        prep,
        state,
        dstate,
        {l2 ? (const void*)gdn_bwd_dqkw_kernel<T, 1, true> : (const void*)gdn_bwd_dqkw_kernel<T, KT>, bwd_dqkw_smem<KT>(), "gdn_bwd_dqkw_kernel", units < 256u ? units : 256u},
        wy,
    };
    for (int i = 0; i < 5; ++i) {
        if (ks[i].grid == 0) continue;
        if (int rc = ensure_dynamic_smem_for(ks[i].f, ks[i].smem, ks[i].name)) return rc;
        void* args[] = {(void*)&p, (void*)&second_arg[i]};
        if (hipLaunchKernel(ks[i].f, dim3(ks[i].grid), dim3(threads[i]), args, ks[i].smem, stream) != hipSuccess) return check_launch(ks[i].name);
        if (int rc = check_launch(ks[i].name)) return rc;
    }
    return GDN_OK;
}

#include "gdn_chunk_kda_bwd.h"      // (inside the namespace: it builds on the types and the two scans above)

}  // namespace gdn

extern "C" size_t gdn_chunk_bwd_workspace_bytes(int64_t num_chunks, int64_t HV, int64_t K) {
    if (num_chunks < 0 || HV < 1 || (K != 128 && K != 256)) return 0;
    return gdn::bwd_ws_layout(num_chunks * HV, K, nullptr, nullptr);
}

// Both operators' entry: `pk` (and `dp`) non-NULL selects comba.
static int chunk_bwd_entry(
    const char* who, bool comba, bool l2,
    const void* q, const void* k, const void* pk, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dp, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    using namespace gdn;
    GDN_CHECK_ARG(B >= 1 && T >= 0 && H >= 1 && HV >= 1 && N >= 1 && num_chunks >= 0, GDN_ERR_INVALID, "%s: bad dimension", who);
    GDN_CHECK_ARG(HV % H == 0, GDN_ERR_INVALID, "%s: HV=%lld not divisible by H=%lld", who, (long long)HV, (long long)H);
    GDN_CHECK_ARG((K == BD || (K == 2 * BD && !comba)) && V == BD, GDN_ERR_UNSUPPORTED,
                  "%s: K = 128%s and V = 128 only (got K=%lld V=%lld); pad smaller head dims with zeros", who, comba ? "" : " or 256",
                  (long long)K, (long long)V);
    GDN_CHECK_ARG(qkv_dtype == GDN_DTYPE_BF16 || qkv_dtype == GDN_DTYPE_F16, GDN_ERR_UNSUPPORTED, "%s: q/k/v/do must be bf16 or f16", who);
    GDN_CHECK_ARG((flags & ~(uint32_t)(GDN_FLAG_CU_INT32 | GDN_FLAG_SCAN_WIDE | GDN_FLAG_SCAN_SEGMENTS)) == 0, GDN_ERR_UNSUPPORTED,
                  "%s: only GDN_FLAG_CU_INT32 and the two flags that steer the scans' time segments are understood here (activations and the state layout are the caller's)", who);
    GDN_CHECK_ARG(HV <= 65535 && num_chunks * HV < (1ll << 31) && N * HV * 4 < (1ll << 31), GDN_ERR_UNSUPPORTED,
                  "%s: too many heads or chunks for one launch", who);
    if (cu_seqlens) {
        GDN_CHECK_ARG(B == 1, GDN_ERR_INVALID, "%s: with cu_seqlens B must be 1", who);
        GDN_CHECK_ARG((chunk_table || num_chunks == 0) && chunk_offsets, GDN_ERR_INVALID, "%s: packed input needs chunk_table and chunk_offsets", who);
    } else {
        GDN_CHECK_ARG(N == B, GDN_ERR_INVALID, "%s: without cu_seqlens N must equal B", who);
        GDN_CHECK_ARG(num_chunks == B * ((T + CH - 1) / CH), GDN_ERR_INVALID, "%s: num_chunks does not match B and T", who);
    }
    hipStream_t s = (hipStream_t)stream;
    if (T == 0 || num_chunks == 0) {
        if (dh0) return launch_state_copy(dht, dh0, N * HV * K * V, s);
        return GDN_OK;
    }
    GDN_CHECK_ARG(q && k && v && beta && dout && dq && dk && dv && dg && dbeta, GDN_ERR_INVALID,
                  "%s: q, k, v, beta, do, dq, dk, dv, dg, dbeta must not be NULL", who);
    GDN_CHECK_ARG(!comba || (pk && dp && g), GDN_ERR_INVALID, "%s: p, g and dp must not be NULL", who);
    GDN_CHECK_ARG(!l2 || (H == HV && K == BD), GDN_ERR_UNSUPPORTED,
                  "%s: the l2 normalisation is taken in here for H == HV and K = 128 only", who);
    for (const void* x : {q, k, pk, v, dout, (const void*)h0, (const void*)dht, (const void*)dq, (const void*)dk, (const void*)dp, (const void*)dv, (const void*)dh0})
        GDN_CHECK_ARG(((uintptr_t)x % 16) == 0, GDN_ERR_INVALID, "%s: tensors must be 16-byte aligned", who);
    GDN_CHECK_ARG(((uintptr_t)workspace % 256) == 0, GDN_ERR_INVALID, "%s: the workspace must be 256-byte aligned", who);
    BwdParams p;
    size_t need = bwd_ws_layout(num_chunks * HV, K, (char*)workspace, &p.ws);
    const size_t rows_bytes = ws_align((size_t)(B * T * H) * BD * 2), factors_bytes = ws_align((size_t)(B * T * H) * 4);
    const size_t l2_at = need;
    if (l2) need += (comba ? 3 : 2) * (rows_bytes + factors_bytes);
    GDN_CHECK_ARG(workspace && workspace_bytes >= need, GDN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who,
                  need, workspace_bytes);
    p.q_raw = p.k_raw = p.pk_raw = nullptr; p.q_rstd = p.k_rstd = p.p_rstd = nullptr;
    if (l2) {
        char* at = (char*)workspace + l2_at;
        p.q_raw = q; p.k_raw = k;
        q = at; k = at + rows_bytes;
        p.q_rstd = (const float*)(at + 2 * rows_bytes); p.k_rstd = (const float*)(at + 2 * rows_bytes + factors_bytes);
        if (comba) {
            at += 2 * (rows_bytes + factors_bytes);
            p.pk_raw = pk;
            pk = at;
            p.p_rstd = (const float*)(at + rows_bytes);
        }
    }
    p.q = q; p.k = k; p.v = v; p.g = g; p.beta = beta; p.h0 = h0; p.dout = dout; p.dht = dht;
    p.dq = dq; p.dk = dk; p.dv = dv; p.dg = dg; p.dbeta = dbeta; p.dh0 = dh0; p.pk = pk; p.dp = dp; p.dgk = nullptr;
    p.cu_seqlens = cu_seqlens; p.chunk_table = chunk_table; p.chunk_offsets = chunk_offsets;
    p.T = T; p.H = (int)H; p.HV = (int)HV; p.N = N; p.NT = (T + CH - 1) / CH;
    p.scale = scale; p.gb_dtype = gb_dtype; p.flags = flags;
    p.nseg = 1; p.seg_chunks = (int)p.NT; p.warm_cap = 0;
    if (comba) return qkv_dtype == GDN_DTYPE_BF16 ? launch_bwd<bf16_t, 1, true>(p, num_chunks, s) : launch_bwd<f16_t, 1, true>(p, num_chunks, s);
    if (K == BD) return qkv_dtype == GDN_DTYPE_BF16 ? launch_bwd<bf16_t, 1>(p, num_chunks, s) : launch_bwd<f16_t, 1>(p, num_chunks, s);
    return qkv_dtype == GDN_DTYPE_BF16 ? launch_bwd<bf16_t, 2>(p, num_chunks, s) : launch_bwd<f16_t, 2>(p, num_chunks, s);
}

extern "C" int gdn_chunk_bwd(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    return chunk_bwd_entry("gdn_chunk_bwd", false, false, q, k, nullptr, v, g, beta, h0, dout, dht, dq, dk, nullptr, dv, dg, dbeta, dh0,
                           cu_seqlens, chunk_table, chunk_offsets, workspace, workspace_bytes, B, T, H, HV, K, V, N, num_chunks,
                           scale, qkv_dtype, gb_dtype, flags, stream);
}

extern "C" size_t gdn_chunk_bwd_qk_l2norm_workspace_bytes(int64_t num_chunks, int64_t HV, int64_t K, int64_t tokens) {
    if (num_chunks < 0 || HV < 1 || K != 128 || tokens < 0) return 0;
    return gdn::bwd_ws_layout(num_chunks * HV, K, nullptr, nullptr) + 2 * gdn::ws_align((size_t)(tokens * HV) * gdn::BD * 2) +
           2 * gdn::ws_align((size_t)(tokens * HV) * 4);
}

extern "C" int gdn_chunk_bwd_qk_l2norm(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    return chunk_bwd_entry("gdn_chunk_bwd_qk_l2norm", false, true, q, k, nullptr, v, g, beta, h0, dout, dht, dq, dk, nullptr, dv, dg, dbeta, dh0,
                           cu_seqlens, chunk_table, chunk_offsets, workspace, workspace_bytes, B, T, H, HV, K, V, N, num_chunks,
                           scale, qkv_dtype, gb_dtype, flags, stream);
}

extern "C" int gdn_chunk_comba_bwd(
    const void* q, const void* k, const void* p, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dp, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    return chunk_bwd_entry("gdn_chunk_comba_bwd", true, false, q, k, p, v, g, beta, h0, dout, dht, dq, dk, dp, dv, dg, dbeta, dh0,
                           cu_seqlens, chunk_table, chunk_offsets, workspace, workspace_bytes, B, T, H, HV, K, V, N, num_chunks,
                           scale, qkv_dtype, gb_dtype, flags, stream);
}

extern "C" size_t gdn_chunk_comba_bwd_qk_l2norm_workspace_bytes(int64_t num_chunks, int64_t HV, int64_t tokens) {
    if (num_chunks < 0 || HV < 1 || tokens < 0) return 0;
    return gdn::bwd_ws_layout(num_chunks * HV, gdn::BD, nullptr, nullptr) + 3 * gdn::ws_align((size_t)(tokens * HV) * gdn::BD * 2) +
           3 * gdn::ws_align((size_t)(tokens * HV) * 4);
}

extern "C" int gdn_chunk_comba_bwd_qk_l2norm(
    const void* q, const void* k, const void* p, const void* v, const void* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dp, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    return chunk_bwd_entry("gdn_chunk_comba_bwd_qk_l2norm", true, true, q, k, p, v, g, beta, h0, dout, dht, dq, dk, dp, dv, dg, dbeta, dh0,
                           cu_seqlens, chunk_table, chunk_offsets, workspace, workspace_bytes, B, T, H, HV, K, V, N, num_chunks,
                           scale, qkv_dtype, gb_dtype, flags, stream);
}

extern "C" size_t gdn_chunk_kda_bwd_workspace_bytes(int64_t num_chunks, int64_t HV) {
    if (num_chunks < 0 || HV < 1) return 0;
    return gdn::kda_bwd_ws_layout(num_chunks * HV, nullptr, nullptr);
}

extern "C" int gdn_chunk_kda_bwd(
    const void* q, const void* k, const void* v, const float* g, const void* beta,
    const float* h0, const void* dout, const float* dht,
    void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    using namespace gdn;
    const char* who = "gdn_chunk_kda_bwd";
    GDN_CHECK_ARG(B >= 1 && T >= 0 && H >= 1 && HV >= 1 && N >= 1 && num_chunks >= 0, GDN_ERR_INVALID, "%s: bad dimension", who);
    GDN_CHECK_ARG(HV % H == 0, GDN_ERR_INVALID, "%s: HV=%lld not divisible by H=%lld", who, (long long)HV, (long long)H);
    GDN_CHECK_ARG(K == BD && V == BD, GDN_ERR_UNSUPPORTED, "%s: K = V = 128 only (got K=%lld V=%lld); pad smaller head dims with zeros",
                  who, (long long)K, (long long)V);
    GDN_CHECK_ARG(qkv_dtype == GDN_DTYPE_BF16 || qkv_dtype == GDN_DTYPE_F16, GDN_ERR_UNSUPPORTED, "%s: q/k/v/do must be bf16 or f16", who);
    GDN_CHECK_ARG((flags & ~(uint32_t)GDN_FLAG_CU_INT32) == 0, GDN_ERR_UNSUPPORTED,
                  "%s: only GDN_FLAG_CU_INT32 is understood here (activations and the state layout are the caller's)", who);
    GDN_CHECK_ARG(HV <= 65535 && num_chunks * HV < (1ll << 31) && N * HV * 4 < (1ll << 31), GDN_ERR_UNSUPPORTED,
                  "%s: too many heads or chunks for one launch", who);
    if (cu_seqlens) {
        GDN_CHECK_ARG(B == 1, GDN_ERR_INVALID, "%s: with cu_seqlens B must be 1", who);
        GDN_CHECK_ARG((chunk_table || num_chunks == 0) && chunk_offsets, GDN_ERR_INVALID, "%s: packed input needs chunk_table and chunk_offsets", who);
    } else {
        GDN_CHECK_ARG(N == B, GDN_ERR_INVALID, "%s: without cu_seqlens N must equal B", who);
        GDN_CHECK_ARG(num_chunks == B * ((T + CH - 1) / CH), GDN_ERR_INVALID, "%s: num_chunks does not match B and T", who);
    }
    hipStream_t s = (hipStream_t)stream;
    if (T == 0 || num_chunks == 0) {
        if (dh0) return launch_state_copy(dht, dh0, N * HV * K * V, s);
        return GDN_OK;
    }
    GDN_CHECK_ARG(q && k && v && g && beta && dout && dq && dk && dv && dg && dbeta, GDN_ERR_INVALID,
                  "%s: q, k, v, g, beta, do, dq, dk, dv, dg, dbeta must not be NULL", who);
    for (const void* x : {q, k, v, dout, (const void*)g, (const void*)h0, (const void*)dht, (const void*)dq, (const void*)dk, (const void*)dv,
                          (const void*)dg, (const void*)dh0})
        GDN_CHECK_ARG(((uintptr_t)x % 16) == 0, GDN_ERR_INVALID, "%s: tensors must be 16-byte aligned", who);
    GDN_CHECK_ARG(((uintptr_t)workspace % 256) == 0, GDN_ERR_INVALID, "%s: the workspace must be 256-byte aligned", who);
    BwdParams p;
    const size_t need = kda_bwd_ws_layout(num_chunks * HV, (char*)workspace, &p.ws);
    GDN_CHECK_ARG(workspace && workspace_bytes >= need, GDN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who,
                  need, workspace_bytes);
    p.q = q; p.k = k; p.v = v; p.g = nullptr; p.beta = beta; p.h0 = h0; p.dout = dout; p.dht = dht;
    p.dq = dq; p.dk = dk; p.dv = dv; p.dg = nullptr; p.dbeta = dbeta; p.dh0 = dh0; p.pk = nullptr; p.dp = nullptr; p.dgk = dg;
    p.q_raw = p.k_raw = p.pk_raw = nullptr; p.q_rstd = p.k_rstd = p.p_rstd = nullptr;
    p.cu_seqlens = cu_seqlens; p.chunk_table = chunk_table; p.chunk_offsets = chunk_offsets;
    p.T = T; p.H = (int)H; p.HV = (int)HV; p.N = N; p.NT = (T + CH - 1) / CH;
    p.scale = scale; p.gb_dtype = gb_dtype; p.flags = flags;
    p.nseg = 1; p.seg_chunks = (int)p.NT; p.warm_cap = 0;
    // the forward's chunk-parallel kernel again, writing into this workspace (u where the scan will put v_new)
    KdaParams kp;
    kp.q = q; kp.k = k; kp.v = v; kp.g = g; kp.beta = beta; kp.pk = nullptr; kp.gs = nullptr;
    kp.A_log = nullptr; kp.gk_bias = nullptr; kp.gk_lower = 0.f; kp.gk_act = 0;
    kp.h0 = nullptr; kp.ht = nullptr; kp.o = nullptr; kp.hs = nullptr;
    kp.cu_seqlens = cu_seqlens; kp.chunk_table = chunk_table; kp.chunk_offsets = chunk_offsets;
    kp.ws = KdaWs{p.ws.Wm, p.ws.Vn, p.ws.QG, p.ws.KG, p.ws.Pm, p.ws.EGL, p.ws.Am, p.ws.Gk};
    kp.T = T; kp.H = (int)H; kp.HV = (int)HV; kp.N = N; kp.NT = p.NT;
    kp.scale = scale; kp.gb_dtype = gb_dtype; kp.flags = flags;
    return qkv_dtype == GDN_DTYPE_BF16 ? launch_bwd_kda<bf16_t>(p, kp, num_chunks, qkv_dtype, s) : launch_bwd_kda<f16_t>(p, kp, num_chunks, qkv_dtype, s);
}
