// Sequential stage of the chunked prefill, two runs per workgroup.
//
// Same mathematics and register layout as gdn_chunk_wide.hip (see there for the formulation,
// the permutation of the state rows and the placement of the q / k tiles in LDS); what differs
// is who does the work.  A compute wave alone on its SIMD spends about half of a step waiting
// (LDS latency, results of the matrix pipeline, barriers), so here every SIMD holds TWO
// compute waves that belong to two independent runs ("teams") reading the same k (and q)
// rows:
//   whole sequences / pass 2   the two value heads 2j, 2j+1 of one q/k head (needs HV/H even)
//   pass 1                     the S run and the M run of one (value head, segment)
// Team tm = wave / 4 owns one 128 x 128 state; wave cw = wave % 4 of a team owns its value
// columns 32cw .. 32cw+31.  Inside a wave the two 16-column tiles interleave in groups of four
// (index i of tile nn is column 32cw + 8*(i/4) + 4*nn + i%4), so that a lane of the transposed
// output tile holds 8 consecutive columns of a token row: one 16-byte store.
//
// There are no copy waves.  Every wave issues its share of the asynchronous global->LDS copies
// (k and q: 2 of the 16 four-row blocks each; its team's record: a quarter; and the 64 bytes
// per token of v that only this wave reads, into an LDS area private to the wave) and stores
// its own output columns straight from registers.  One barrier per chunk publishes the shared
// copies; the private v area needs none.  All copies and stores of a wave complete in issue
// order, so "at most N operations outstanding" proves that everything older has landed; the
// counts below are the number of operations a wave issues after the one it waits for.
#include "gdn_chunk_common.h"

namespace gdn {

// LDS: k and q double-buffered (chunk % 2), records double-buffered per team, v single-buffered
// per wave (each half of the rows is fetched again as soon as the wave has consumed it).
constexpr int PR_K = 0, PR_Q = 32768, PR_V = 65536, PR_REC = 98304;
constexpr int PR_OT = PR_REC + 4 * (int)REC_BYTES;            // 8 x 1 KB: per wave, one 16-token tile of its output columns on its way out
constexpr int PR_PCOUNT = PR_OT + 8 * 1024;                   // per team: P fragments published so far
constexpr size_t PAIR_SMEM = PR_PCOUNT + 16;                  // 151 568 B
constexpr int PAIR_THREADS = 512;

// One 16-byte store per lane at sbase + voff, for the lanes named by `mask` only.  Written in
// assembly so that the address stays a scalar base plus a 32-bit lane offset, and so that exactly
// one operation is issued whatever the mask: the execution mask is narrowed around the store by
// hand instead of by a conditional in the source.
__device__ __forceinline__ void store16_masked(const char* sbase, uint32_t voff, u32x4 d, uint64_t mask) {
    const uint64_t g = (uint64_t)sbase;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)g), hi = __builtin_amdgcn_readfirstlane((uint32_t)(g >> 32));
    const uint64_t gs = ((uint64_t)hi << 32) | lo;
    uint64_t saved;
    asm volatile("s_and_saveexec_b64 %0, %1\n\t"
                 "global_store_dwordx4 %2, %3, %4\n\t"
                 "s_mov_b64 exec, %0"
                 : "=&s"(saved) : "s"(mask), "v"(voff), "v"(d), "s"(gs) : "memory", "scc");
}

template <typename T, bool FULL, bool DIMS128>
__global__ __launch_bounds__(PAIR_THREADS) void gdn_chunk_pair_kernel(ChunkParams p, SegmentPlan sp) {
    // Head dims: DIMS128 fixes K = V = 128 at compile time (every copy is whole, nothing is masked); otherwise they
    // are the caller's multiples of 8 and the tiles' features past them are zero (q, k) or never stored (v, o, state).
    const int K = DIMS128 ? 128 : p.K, V = DIMS128 ? 128 : p.V;
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];

    const int tid = threadIdx.x, lane = tid & 63, c16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tm = w >> 2, cw = w & 3;
    const int H = p.H, HV = p.HV;
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    const bool l2q = p.flags & FLAG_Q_NORM_IN_SCAN;       // q is l2-normalised where P is formed (row factors)
    const bool vfirst = p.flags & GDN_FLAG_STATE_V_FIRST;

    // ---- which runs: workgroups that read the same k rows take consecutive slots of one XCD ----
    const int G = HV / H;
    const int64_t slot = blockIdx.x >> 3;
    const int xcd = blockIdx.x & 7;
    int64_t n;
    int h, hv, seg;
    int init = 0;                 // 0: from `src` (NULL = zero state), 1: identity, 2: zero
    bool v_zero = false, src_user = false, dst_user = false, active = true;
    const float* src = nullptr;
    float* dst = nullptr;
    if (sp.kind == WIDE_WHOLE) {
        const int mem = G >> 1;
        const int64_t group = (slot / mem) * 8 + xcd;                 // (sequence, q/k head)
        if (group >= p.N * H) return;
        n = group / H;
        if (p.flags & GDN_FLAG_SEQ_ORDER) n = load_index(p.chunk_offsets, p.N + 1 + n, cu32);
        h = (int)(group % H); hv = h * G + 2 * (int)(slot % mem) + tm; seg = 0;
        const int64_t inh = n * HV + hv;
        src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true;
        dst = p.ht ? p.ht + inh * (int64_t)(K * V) : nullptr; dst_user = true;
    } else if (sp.kind == WIDE_PASS1) {
        const int64_t group = (slot / G) * 8 + xcd;                   // (sequence, q/k head, segment 0 .. nseg-2)
        if (group >= p.N * H * (sp.nseg - 1)) return;
        const int64_t nh = group / (sp.nseg - 1);
        seg = (int)(group % (sp.nseg - 1));
        n = nh / H; h = (int)(nh % H); hv = h * G + (int)(slot % G);
        const int64_t inh = n * HV + hv;
        // (a head whose segments all start warm needs no exact start states)
        if (sp.bound && !needs_exact_segments(sp, sp.bound + n * p.NT * HV + hv, HV, lane)) return;
        if (tm == 0) {
            if (seg == 0) { src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true; }
            else init = 2;
            dst = sp.sloc + (inh * sp.nseg + seg) * 16384;
        } else {
            if (seg == 0) active = false;                             // the first segment starts from the true state: no transition needed
            init = 1; v_zero = true;
            dst = sp.mseg + (inh * sp.nseg + seg) * 16384;
        }
    } else {
        const int mem = G >> 1;
        const int64_t group = (slot / mem) * 8 + xcd;                 // (sequence, q/k head, segment)
        if (group >= p.N * H * sp.nseg) return;
        const int64_t nh = group / sp.nseg;
        seg = (int)(group % sp.nseg);
        n = nh / H; h = (int)(nh % H); hv = h * G + 2 * (int)(slot % mem) + tm;
        const int64_t inh = n * HV + hv;
        if (seg == 0) { src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true; }
        else src = sp.sin + (inh * sp.nseg + seg) * 16384;
        if (seg == sp.nseg - 1 && p.ht) { dst = p.ht + inh * (int64_t)(K * V); dst_user = true; }
    }

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
    const int64_t it0 = (int64_t)seg * sp.seg_chunks;
    const int64_t it1 = min(nt, it0 + sp.seg_chunks);
    const int64_t nsteps = it1 - it0;                       // may be <= 0 for an empty sequence
    const int64_t lastc = it1 - 1;

    // =====================================================================================
    // Copies.  Rows past the end of the sequence re-read its last row: whatever they hold is
    // finite and is multiplied by the zero columns of Xb, the zero rows of v_new and the causal
    // zeros of P.
    // =====================================================================================
    const bool vz = __builtin_amdgcn_readfirstlane((int)v_zero) != 0;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    // P = scale tril(q k^T 2^(G_t - G_t')) of a chunk is formed by the four waves of a team from the q and k tiles at the
    // start of its step (see gdn_chunk_wide.hip); a counter per team in LDS tells when its fragments are complete.
    volatile int* pcount = (volatile int*)(smem + PR_PCOUNT) + tm;
    if (tid == 0) { ((volatile int*)(smem + PR_PCOUNT))[0] = 0; ((volatile int*)(smem + PR_PCOUNT))[1] = 0; }      // (published by the first barrier)
    // rows of the caller's tensors hold K (q, k) or V (v, o) elements, multiples of 8 up to 128.  Pieces of q and k
    // past K stay zero in LDS (the tiles are cleared once, those lanes copy nothing); pieces of v past V re-read
    // valid ones: value columns never mix, and the padded ones are never stored.
    const uint32_t rowB_qk = (uint32_t)H * K * 2, rowB_v = (uint32_t)HV * V * 2;
    const int k_pieces = K >> 3, v_pieces = V >> 3;
    // k and q tiles in LDS: 64 token rows x 256 B as 16 blocks of 4 rows (1 KB, one copy each).  In block j
    // the 16-byte piece c of row 4j + r sits in slot 16*(c/4) + 4r + ((c + j) & 3): four consecutive lanes
    // fetch 64 contiguous bytes of one row, and both the operand reads (16 rows x one piece) and the
    // transpose reads (4 rows x 4 pieces) of a 16-lane group touch 16 different slots modulo 16.
    // This wave copies blocks 2w and 2w+1: lane -> (row, byte offset of its piece)
    int kq_row[2];
    uint32_t kq_cb[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const int j = 2 * w + e;
        kq_row[e] = 4 * j + (c16 >> 2);
        kq_cb[e] = 16 * (4 * g + ((c16 - j) & 3));
    }
    uint64_t kq_mask[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) kq_mask[e] = __builtin_amdgcn_ballot_w64((int)(kq_cb[e] >> 4) < k_pieces);
    auto issue_kq = [&](const T* tensor, int64_t c, uint32_t lds_tile) {            // 2 operations
        const int valid = (int)min((int64_t)CH, len - c * CH);
        const char* base = (const char*)(tensor + ((bos + c * CH) * H + h) * K);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint32_t row = (uint32_t)min(kq_row[e], valid - 1);
            if constexpr (DIMS128) gather_1k_to_lds(base, __umul24(row, rowB_qk) + kq_cb[e], lds_tile + (2 * w + e) * 1024);
            else gather_1k_to_lds_masked(base, __umul24(row, rowB_qk) + kq_cb[e], lds_tile + (2 * w + e) * 1024, kq_mask[e]);
        }
    };
    // private v area: block b = rows 16b .. 16b+15 x this wave's 4 pieces (64 bytes of a row are
    // fetched by 4 consecutive lanes); piece pc of row r sits in slot 4r + pc, so the transpose reads
    // of a 16-lane group (4 rows x 4 pieces) cover 16 consecutive slots
    const int v_r16 = lane >> 2;
    const uint32_t v_cb = 16 * ((4 * cw + (lane & 3)) % v_pieces);
    auto issue_v = [&](int64_t c, int half) {                                        // 2 operations
        const int valid = v_zero ? 1 : (int)min((int64_t)CH, len - c * CH);         // (a transition run reads no v: one row, from cache)
        const char* base = (const char*)((const T*)p.v + ((bos + c * CH) * HV + hv) * V);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int b = 2 * half + e;
            const uint32_t row = (uint32_t)min(16 * b + v_r16, valid - 1);
            gather_1k_to_lds(base, __umul24(row, rowB_v) + v_cb, lds0 + PR_V + w * 4096 + b * 1024);
        }
    };
    // The record of (chunk, value head), in 1 KB pieces.  A full run needs Xb and the two tables (pieces 0..4, 10, 11: P is
    // formed here), two per wave of the team.  A state-only run needs Xb and the first table (pieces 0..4 and 10), and its two
    // teams work on the same value head: they share one copy (in the area of team 0), one piece per wave.
    auto issue_rec = [&](int64_t c, int stage) {                                     // 2 operations (state-only: 1)
        const char* rec = p.ws.Rec + ((boh + c) * HV + hv) * REC_BYTES;
        const uint32_t to = lds0 + PR_REC + ((FULL ? tm : 0) * 2 + stage) * (uint32_t)REC_BYTES;
        auto piece = [&](int j) { gather_1k_to_lds(rec + j * 1024, lane * 16, to + j * 1024); };
        if constexpr (FULL) {
            piece(cw);                                                                // Xb 0..3
            piece(cw == 0 ? REC_PIECES_X - 1 : cw == 1 ? REC_PIECE_TAB : cw == 2 ? REC_PIECE_TAB2 : 0);      // (wave 3 fetches piece 0 again: equal counts)
        } else {
            piece(w < REC_PIECES_X ? w : w == REC_PIECES_X ? REC_PIECE_TAB : 0);      // (waves 6, 7 fetch piece 0 again: equal counts)
        }
    };
    // everything a barrier publishes, 6 (3) operations, in three parts so that the waves do not all
    // queue at the memory pipeline at once
    auto issue_shared = [&](int64_t c, int stage, int part) {
        if (part == 0) issue_kq((const T*)p.k, c, lds0 + PR_K + stage * 16384);
        if (part == 1) { if constexpr (FULL) issue_kq((const T*)p.q, c, lds0 + PR_Q + stage * 16384); }
        if (part == 2) issue_rec(c, stage);
    };
    // number of operations a wave issues between ...
    // (per step, in order: shared 6 (3), in the first three regions | v rows 0..31: 2 | output tiles 0, 1: 2 | v rows 32..63: 2 | output tiles 2, 3: 2)
    constexpr int N_AFTER_SHARED = FULL ? 8 : 4;      // the shared copies of a step and the barrier at its end
    constexpr int N_AFTER_VLO = FULL ? 12 : 5;        // the first half of v and its use in the next step
    constexpr int N_AFTER_VHI = FULL ? 10 : 5;        // the second half of v and its use in the next step

    if (K < 128 && nsteps > 0) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int i = tid; i < (PR_V - PR_K) / 16; i += PAIR_THREADS) *(u32x4*)(smem + PR_K + i * 16) = z;
        lds_barrier();
    }
    if (nsteps > 0 && !active) {
        // a team with nothing to compute still fetches its share of k and of the record
        issue_kq((const T*)p.k, it0, lds0 + PR_K);
        issue_rec(it0, 0);
        wait_vm_at_most<0>();
        lds_barrier();
        for (int64_t i = 0; i < nsteps; ++i) {
            issue_kq((const T*)p.k, min(it0 + i + 1, lastc), lds0 + PR_K + (int)((i + 1) & 1) * 16384);
            issue_rec(min(it0 + i + 1, lastc), (int)((i + 1) & 1));
            wait_vm_at_most<0>();
            lds_barrier();
        }
        return;
    }
    if (!active) return;

    // ---- state: all key rows (permuted), value columns 32cw .. 32cw+31, C/D layout ----
    constexpr int NN = 2;
    f32x4 S[8][NN];
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
    for (int nn = 0; nn < NN; ++nn) {
        const int kk = 32 * (m >> 1) + 8 * g + 4 * (m & 1), vc = 32 * cw + 8 * (c16 >> 2) + 4 * nn + (c16 & 3);
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        if (init == 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] = (kk + r == vc) ? 1.f : 0.f;
        } else if (init == 0 && src) {
            // the caller's state is [K][V] or [V][K] with rows and columns past K, V counting as zero; the buffers
            // of the segment passes are [128][128]: one strided form serves all three
            const int sk = src_user ? (vfirst ? 1 : V) : 128, sv = src_user ? (vfirst ? K : 1) : 1;
            if (kk < (src_user ? K : 128) && vc < (src_user ? V : 128)) {
                const float* e = src + kk * sk + vc * sv;
                s = f32x4{e[0], e[sk], e[2 * sk], e[3 * sk]};
            }
        }
        S[m][nn] = s;
    }

    // lazy decay: the registers hold S / Gamma, Gamma = 2^lg (see gdn_chunk_wide.hip)
    constexpr float LG_MIN = std::is_same<T, bf16_t>::value ? -60.f : 1.f;
    float lg = 0.f;

    const int tr_i = c16 >> 2, tr_j = c16 & 3;
    const int a_off = (c16 >> 2) * 64 + 4 * (c16 & 3) + ((g + (c16 >> 2)) & 3);     // operand piece 4s + g of row c16 of a t-tile: + tt*256 + 16*s  (16-byte units)
    const int k_tr = (g * 64 + 4 * tr_i + ((tr_j + g) & 3)) * 8;                    // row 4g+i of a 16-row group, piece 4*(m/2) + j: + (32*sp2 + 16*half)*128 + 128*(m/2) + 4*(m&1)  (elements)
    const int v_tr = (4 * (4 * g + tr_i) + tr_j) * 8;                     // private v area: row 4g + i of a block, piece j: + 4*nn + tt*512  (elements)
    // Output: a lane of the transposed tile holds token row c16, 8 value columns (piece g of the wave's
    // 64 bytes of that row).  Stored like that, neighbouring lanes would write to different rows, which
    // the memory pipeline handles one lane at a time; so the tile takes a turn through a private LDS
    // area (slot 4*row + ((piece + row/4) & 3): conflict-free both ways) and leaves with lane l holding
    // row l/4, i.e. four consecutive lanes writing 64 contiguous bytes.
    char* ot = smem + PR_OT + w * 1024;
    const int ot_w = (4 * c16 + ((g + (c16 >> 2)) & 3)) * 16;
    const int o_row = lane >> 2;
    const int o_piece = 4 * cw + (((lane & 3) - (o_row >> 2)) & 3);        // 16-byte piece of the output row this lane stores
    const uint32_t o_voff = (uint32_t)o_row * rowB_v + 16 * o_piece;

    // One step: the regions of the four-wave kernel, plus this wave's copies and stores.
    auto step = [&](int64_t i) {
        const int cur = (int)(i & 1);
        const int64_t it = it0 + i;
        const char* kbuf = smem + PR_K + cur * 16384;
        const V8* sK = (const V8*)kbuf;
        const V8* sQ = (const V8*)(smem + PR_Q + cur * 16384);
        const T* sV = (const T*)(smem + PR_V + w * 4096);
        const T* sKt = (const T*)kbuf;
        const char* rec = smem + PR_REC + ((FULL ? tm : 0) * 2 + cur) * REC_BYTES;
        const char* sX = rec + REC_X;
        const char* sP = rec + REC_P;
        const float* sTab = (const float*)(rec + REC_TAB);
        const char* obase = (const char*)p.o + ((bos + it * CH) * HV + hv) * (int64_t)(V * 2);
        const int valid = (int)min((int64_t)CH, len - it * CH);
        auto fence = [] { __builtin_amdgcn_sched_barrier(0); };

        const int64_t nxt = min(it + 1, lastc);                 // (its buffers were released by the barrier that ended the previous step)

        if constexpr (FULL) {
            // ---- this wave's share of P (transposed product, so that a result is spread over the lanes like the operand
            // fragment that is read back), gated with its team's tables ----
            const float* t2 = (const float*)(rec + REC_TAB2);
            auto frag = [&](int tt, int sp) {
                V8 qb[4];
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) qb[s4] = sQ[tt * 256 + 16 * s4 + a_off];
                const int t = 16 * tt + c16;
                float gt = t2[TAB2_G + t], st_ = t2[TAB2_NQS + t];
                if (l2q) {                        // q is normalised here: P, and the table that scales the (q S) rows
                    const float nq = row_rnorm<T>(qb, c16);
                    st_ *= nq;
                    if (sp == 0 && g == 0) ((float*)(rec + REC_TAB))[TAB_SG + t] *= nq;
                }
                V8 out;
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int tj = 2 * sp + half;
                    if (tj > tt) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) out[half * 4 + r] = from_f32<T>(0.f);
                        continue;
                    }
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4) acc = Mma<T>::run(sK[tj * 256 + 16 * s4 + a_off], qb[s4], acc);
                    const f32x4 gj = *(const f32x4*)(t2 + TAB2_G + 16 * tj + 4 * g), nj = *(const f32x4*)(t2 + TAB2_NK + 16 * tj + 4 * g);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int j = 16 * tj + 4 * g + r;
                        // select, never multiply by a mask: 2^(G_t - G_j) may overflow above the diagonal
                        out[half * 4 + r] = from_f32<T>((t >= j) ? st_ * nj[r] * acc[r] * fast_exp2(gt - gj[r]) : 0.f);
                    }
                }
                store_frag<T>((char*)rec + REC_P, tt, sp, lane, out);
            };
            if (cw == 0) frag(3, 0);
            else if (cw == 1) frag(3, 1);
            else if (cw == 2) { frag(2, 0); frag(0, 0); }
            else { frag(1, 0); frag(2, 1); }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0) __hip_atomic_fetch_add((int*)pcount, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            fence();
        }

        constexpr int RING = 2;
        V8 ak[RING], aq[RING];
        auto F = [&](int f) {
            ak[f % RING] = sK[(f >> 2) * 256 + 16 * (f & 3) + a_off];
            if constexpr (FULL) aq[f % RING] = sQ[(f >> 2) * 256 + 16 * (f & 3) + a_off];
        };
        f32x4 ks[4][NN], ao[4][NN];
        V8 Sb[4][NN];
        auto M = [&](int f) {
            const int tt = f >> 2, sx = f & 3;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) {
                ks[tt][nn] = Mma<T>::run(ak[f % RING], Sb[sx][nn], sx ? ks[tt][nn] : f32x4{0.f, 0.f, 0.f, 0.f});
                if constexpr (FULL) ao[tt][nn] = Mma<T>::run(Sb[sx][nn], aq[f % RING], sx ? ao[tt][nn] : f32x4{0.f, 0.f, 0.f, 0.f});
            }
        };
        V4 vv[4][NN];
        V8 ax[4][2], ap[4][2];
        auto FV = [&](int tt) {
            if (!FULL && vz) return;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) vv[tt][nn] = Mma<T>::tr_read(sV + tt * 512 + v_tr + 4 * nn);
        };
        auto FX = [&](int tt) {
#pragma unroll
            for (int sp2 = 0; sp2 <= (tt >> 1); ++sp2) ax[tt][sp2] = load_frag<T>(sX, tt, sp2, lane);
        };
        auto FP = [&](int tt) {
            if constexpr (FULL) {
#pragma unroll
                for (int sp2 = 0; sp2 <= (tt >> 1); ++sp2) ap[tt][sp2] = load_frag<T>(sP, tt, sp2, lane);
            }
        };
        V8 kt[2][8];
        auto FK = [&](int sp2, int m) {
            const T* a = sKt + sp2 * 4096 + 128 * (m >> 1) + 4 * (m & 1) + k_tr;
            kt[sp2][m] = join<V8>(Mma<T>::tr_read(a), Mma<T>::tr_read(a + 2048));
        };
        float gamma, vscale;
        V8 Db[2][NN], Vn[2][NN], Vg[2][NN];
        auto TD = [&](int tt) {
            const f32x4 eg = *(const f32x4*)(sTab + TAB_EG + 16 * tt + 4 * g) * gamma;
            if (!FULL && vz) {                  // a transition run has v = 0 (scalar branch: nothing is selected per element)
#pragma unroll
                for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                    for (int r = 0; r < 4; ++r) Db[tt >> 1][nn][(tt & 1) * 4 + r] = from_f32<T>(-eg[r] * ks[tt][nn][r]);
            } else {
#pragma unroll
                for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        Db[tt >> 1][nn][(tt & 1) * 4 + r] = from_f32<T>(to_f32(vv[tt][nn][r]) - eg[r] * ks[tt][nn][r]);
            }
        };
        f32x4 vn[4][NN], oacc[4][NN];
        auto TXa = [&](int tt) {
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) {
                vn[tt][nn] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int sp2 = 0; sp2 <= (tt >> 1); ++sp2) vn[tt][nn] = Mma<T>::run(ax[tt][sp2], Db[sp2][nn], vn[tt][nn]);
            }
        };
        auto TXb = [&](int tt) {
            const f32x4 dec = *(const f32x4*)(sTab + TAB_DEC + 16 * tt + 4 * g) * vscale;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    Vn[tt >> 1][nn][(tt & 1) * 4 + r] = from_f32<T>(vn[tt][nn][r]);
                    Vg[tt >> 1][nn][(tt & 1) * 4 + r] = from_f32<T>(vn[tt][nn][r] * dec[r]);
                }
        };
        auto TPa = [&](int tt) {
            if constexpr (FULL) {
                const float gam = sTab[TAB_SG + 16 * tt + c16] * gamma;
#pragma unroll
                for (int nn = 0; nn < NN; ++nn) {
                    oacc[tt][nn] = ao[tt][nn] * gam;
#pragma unroll
                    for (int sp2 = 0; sp2 <= (tt >> 1); ++sp2) oacc[tt][nn] = Mma<T>::run(Vn[sp2][nn], ap[tt][sp2], oacc[tt][nn]);
                }
            }
        };
        auto TPb = [&](int tt) {                // 1 store: 8 consecutive value columns of a token row per lane
            if constexpr (FULL) {
                V4 o4[NN];
#pragma unroll
                for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                    for (int r = 0; r < 4; ++r) o4[nn][r] = from_f32<T>(oacc[tt][nn][r]);
                const char* ob = obase + (size_t)(16 * tt) * rowB_v;
                const u32x2 lo = __builtin_bit_cast(u32x2, o4[0]), hi = __builtin_bit_cast(u32x2, o4[1]);
                *(u32x4*)(ot + ot_w) = u32x4{lo[0], lo[1], hi[0], hi[1]};
                const u32x4 orow = *(const u32x4*)(ot + lane * 16);       // (LDS operations of a wave execute in order)
                store16_masked(ob, o_voff, orow, __builtin_amdgcn_ballot_w64(16 * tt + o_row < valid && o_piece < v_pieces));
            }
        };
        auto U = [&](int sp2, int m) {
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) S[m][nn] = Mma<T>::run(kt[sp2][m], Vg[sp2][nn], S[m][nn]);
        };

#pragma unroll
        for (int f = 0; f < RING - 1; ++f) F(f);
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    Sb[s][nn][r] = from_f32<T>(S[2 * s][nn][r]);
                    Sb[s][nn][4 + r] = from_f32<T>(S[2 * s + 1][nn][r]);
                }
        gamma = fast_exp2(lg);
        const float lg_try = lg + sTab[TAB_GLAST];
        const bool lazy = lg_try >= LG_MIN;
        vscale = lazy ? fast_exp2(-lg_try) : 1.f;
        fence();
#pragma unroll
        for (int f = 0; f < 16; ++f) {
            if (f + RING - 1 < 16) F(f + RING - 1);
            M(f);
            if (f < 3) issue_shared(nxt, cur ^ 1, f);
            if (f == 4) { wait_vm_at_most<N_AFTER_VLO>(); FV(0); }
            if (f == 5) FV(1);
            if (f == 6) FX(0);
            if (f == 7) FX(1);
            if (f == 8) TD(0);
            if (f == 9) {
                if constexpr (FULL) { while (*pcount < 4 * ((int)i + 1)) __builtin_amdgcn_s_sleep(1); }       // the team's P (long there)
                TD(1); FP(0);
            }
            if (f == 10) { TXa(0); TXa(1); FP(1); issue_v(nxt, 0); }     // (v rows 0..31 are in registers since region 9)
            if (f == 11) { TXb(0); TXb(1); wait_vm_at_most<N_AFTER_VHI>(); FV(2); }
            if (f == 12) { TPa(0); TPa(1); FV(3); }
            if (f == 13) { TPb(0); TPb(1); FX(2); }
            if (f == 14) { FX(3); FK(0, 0); FK(0, 1); }
            if (f == 15) { FK(0, 2); FK(0, 3); }
            fence();
        }
        if (__builtin_amdgcn_readfirstlane((int)lazy) == 0) {
            const float fold = fast_exp2(lg_try);
#pragma unroll
            for (int m = 0; m < 8; ++m)
#pragma unroll
                for (int nn = 0; nn < NN; ++nn) S[m][nn] *= fold;
        }
        lg = lazy ? lg_try : 0.f;
        U(0, 0); U(0, 1); TD(2); FK(0, 4); FK(0, 5); fence();
        U(0, 2); U(0, 3); TD(3); FK(0, 6); FK(0, 7); FP(2); fence();
        U(0, 4); U(0, 5); TXa(2); TXa(3); FK(1, 0); FK(1, 1); FP(3); issue_v(nxt, 1); fence();
        U(0, 6); U(0, 7); TXb(2); TXb(3); FK(1, 2); FK(1, 3); fence();
        U(1, 0); U(1, 1); TPa(2); TPa(3); FK(1, 4); FK(1, 5); fence();
        U(1, 2); U(1, 3); TPb(2); TPb(3); FK(1, 6); FK(1, 7); fence();
        wait_vm_at_most<N_AFTER_SHARED>();                       // this wave's shared copies for the next step have landed
        lds_barrier();                                           // every wave is done reading this step's buffers, the next step's are complete
#pragma unroll
        for (int m = 4; m < 8; ++m) U(1, m);
        fence();
    };

    if (nsteps > 0) {
#pragma unroll
        for (int part = 0; part < 3; ++part) issue_shared(it0, 0, part);
        issue_v(it0, 0);
        issue_v(it0, 1);
        wait_vm_at_most<0>();
        lds_barrier();
        for (int64_t i = 0; i < nsteps; ++i) step(i);
        wait_vm_at_most<0>();                                    // no copy may land in LDS after this workgroup has gone
    }

    if (dst) {
        const float gamma = fast_exp2(lg);
#pragma unroll
        for (int m = 0; m < 8; ++m)
#pragma unroll
        for (int nn = 0; nn < NN; ++nn) {
            const int kk = 32 * (m >> 1) + 8 * g + 4 * (m & 1), vc = 32 * cw + 8 * (c16 >> 2) + 4 * nn + (c16 & 3);
            const f32x4 s = S[m][nn] * gamma;
            const int sk = dst_user ? (vfirst ? 1 : V) : 128, sv = dst_user ? (vfirst ? K : 1) : 1;
            if (kk < (dst_user ? K : 128) && vc < (dst_user ? V : 128)) {
                float* e = dst + kk * sk + vc * sv;
#pragma unroll
                for (int r = 0; r < 4; ++r) e[r * sk] = s[r];
            }
        }
    }
}

template <typename T, bool FULL, bool DIMS128>
static int launch_pair_dims(const ChunkParams& p, const SegmentPlan& sp, int64_t blocks, hipStream_t stream) {
    auto kern = gdn_chunk_pair_kernel<T, FULL, DIMS128>;
    static SmemAttrDone attr_done;       // per instantiation
    if (int rc = ensure_dynamic_smem((const void*)kern, PAIR_SMEM, attr_done, "hipFuncSetAttribute(pair)")) return rc;
    if (blocks <= 0) return GDN_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(PAIR_THREADS), PAIR_SMEM, stream, p, sp);
    return check_launch("gdn_chunk_pair_kernel");
}

template <typename T, bool FULL>
static int launch_pair_kind(const ChunkParams& p, const SegmentPlan& sp, int64_t blocks, hipStream_t stream) {
    return p.K == 128 && p.V == 128 ? launch_pair_dims<T, FULL, true>(p, sp, blocks, stream)
                                    : launch_pair_dims<T, FULL, false>(p, sp, blocks, stream);
}

// sp.kind selects the work: whole sequences and pass 2 need an even number of value heads per
// q/k head; pass 1 pairs the two runs of one value head and works for any head count.
template <typename T>
int launch_pair(const ChunkParams& p, SegmentPlan sp, hipStream_t stream) {
    const int64_t G = p.HV / p.H;
    if (sp.kind == WIDE_PASS1)
        return launch_pair_kind<T, false>(p, sp, (p.N * p.H * (sp.nseg - 1) + 7) / 8 * 8 * G, stream);
    if (G % 2) return GDN_ERR_INVALID;
    if (sp.kind == WIDE_WHOLE) {
        sp.nseg = 1;
        sp.seg_chunks = 1 << 30;
        return launch_pair_kind<T, true>(p, sp, (p.N * p.H + 7) / 8 * 8 * (G / 2), stream);
    }
    return launch_pair_kind<T, true>(p, sp, (p.N * p.H * sp.nseg + 7) / 8 * 8 * (G / 2), stream);
}

template int launch_pair<bf16_t>(const ChunkParams&, SegmentPlan, hipStream_t);
template int launch_pair<f16_t>(const ChunkParams&, SegmentPlan, hipStream_t);

}  // namespace gdn
