// Sequential stage of the chunked prefill: one workgroup per (sequence, v-head, segment of
// consecutive chunks) holds the WHOLE fp32 state S[128, 128] in registers and walks the
// chunks in order.  Per chunk, with Xb = (I+L)^-1 diag(beta), P and the gate tables from the
// prepare kernel and the raw q, k, v tiles:
//   D     = v - 2^G (k S)                      (the delta-rule residual of every token)
//   v_new = Xb D                               (== u - w S of the WY form)
//   o     = scale 2^G (q S) + P v_new
//   S     = 2^G_last S + k^T (v_new 2^(G_last-G))
//
// Eight waves.  Four compute waves, one per SIMD: wave w owns value columns 32w .. 32w+31 for all key
// rows, so every operand fragment read from LDS feeds two matrix instructions.  Nothing of the recurrence crosses waves: bf16(S), bf16(D) and bf16(v_new) are the B
// operands of this wave's own next products (same lanes, C/D layout == operand layout), so
// the dependent chain runs in registers.  The compute waves issue no global memory instruction
// inside the loop.
// Four copy waves move everything else.  Three of them fill a double-buffered LDS stage with
// asynchronous global->LDS loads that use no registers: the prepare record verbatim, and the
// q, k, v tiles gathered straight from the user's tensors in 16-byte pieces, placed so that
// the matrix-core operands are conflict-free 16-byte LDS reads (q, k rows) or LDS transpose
// reads (k^T, v).  The fourth moves the output tile of a chunk LDS -> registers -> global in
// 256-byte rows.  Two barriers per chunk (after each half of a step) are the only
// synchronisation.
//
// State rows are permuted inside the registers so that the 8 contraction indices a lane
// feeds to the matrix core are 8 CONSECUTIVE key features (one 16-byte piece of a q or k
// row): tile m, row 4g+r holds key feature 32*(m/2) + 8g + 4*(m%2) + r.
//
// The same kernel serves the segment-parallel evaluation of long sequences
// (S_out = M S_in + S_loc per segment):
//   pass 1  state only (no q / P / output), started from the true initial state (first
//           segment), from zero (S_loc) or from the identity with v = 0 (the transition M);
//   merge   S_in[j+1] = M_j S_in[j] + S_loc,j in fp32 (gdn_segment_merge_kernel);
//   pass 2  full evaluation of every segment from its merged initial state.
#include "gdn_chunk_common.h"

namespace gdn {

// LDS stage of one chunk.  q, k, v tiles: 64 token rows x 256 B as 16 blocks of 4 rows (1 KB, one
// asynchronous copy each: 4 whole rows is the access shape the memory pipeline moves fastest).
// Inside block j the 16-byte piece c of row 4j + r sits in slot 16*(c/4) + 4r + ((c + j) & 3): four consecutive
// lanes of a copy fetch 64 contiguous bytes of one row (neighbouring lanes on different rows would go through
// the memory pipeline one lane at a time), and the rotation makes both the 16-byte operand reads (16 rows x
// one piece) and the LDS transpose reads (4 rows x 4 pieces) of a 16-lane group touch 16 different slots
// modulo 16, i.e. all banks.
// q, v and the record are double-buffered (stage = chunk % 2); k, the one operand that is read until the
// very end of a step, has three buffers (chunk % 3) so that its copy can be issued two steps ahead.
constexpr int STG_Q = 0, STG_V = 16384, STG_REC = 32768;
constexpr int STG_X = STG_REC + REC_X, STG_P = STG_REC + REC_P, STG_TAB = STG_REC + REC_TAB, STG_TAB2 = STG_REC + REC_TAB2;
constexpr int STG_BYTES = STG_REC + (int)REC_BYTES;          // 45 056
constexpr int KBUF = 2 * STG_BYTES;                          // three k tiles of 16 KB follow the two stages
constexpr int OT_PITCH = 272;                     // bytes per token row of the output tile (256 B + pad: conflict-free 8-byte writes)
constexpr int OT_BYTES = 64 * OT_PITCH;           // 17 408 B
constexpr int PCOUNT_OFF = KBUF + 3 * 16384 + OT_BYTES;       // one counter: P fragments published so far
constexpr size_t WIDE_SMEM = PCOUNT_OFF + 16;                // 156 688 B of the CU's 163 840: one workgroup per CU
constexpr int WIDE_NN = 2;                        // 16-column tiles per compute wave
#ifndef WIDE_RING
#define WIDE_RING 3                               // operand fragments in flight per compute wave
#endif
constexpr int CW = 8 / WIDE_NN;                   // compute waves
constexpr int WIDE_THREADS = (CW + 4) * 64;

template <typename T, bool FULL, bool DIMS128, bool SMALL>
__global__ __launch_bounds__(WIDE_THREADS) void gdn_chunk_wide_kernel(ChunkParams p, SegmentPlan sp) {
    // Head dims: DIMS128 fixes K = V = 128 at compile time (every copy is whole, nothing is masked); otherwise they
    // are the caller's multiples of 8 and the tiles' features past them are zero (q, k) or never stored (v, o, state).
    // SMALL (K, V <= 64, e.g. the reference's D = 64 shapes): a quarter of the state - 64 key rows, 16 value columns
    // per compute wave - with the LDS layout unchanged, so that nothing is multiplied by the zero features.
    static_assert(!(DIMS128 && SMALL), "one or the other");
    const int K = DIMS128 ? 128 : p.K, V = DIMS128 ? 128 : p.V;
    constexpr int KS = SMALL ? 2 : 4;                 // pairs of 16-row key tiles (32 key features each)
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];

    const int tid = threadIdx.x, lane = tid & 63, c16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);       // scalar: the roles below branch on it
    const int H = p.H, HV = p.HV;
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    const bool l2q = p.flags & FLAG_Q_NORM_IN_SCAN;       // q is l2-normalised where P is formed (row factors)
    const bool vfirst = p.flags & GDN_FLAG_STATE_V_FIRST;

    // ---- which (sequence, head, segment) and what to start from / write to ----
    // Workgroups that read the same k (and q) rows - the value heads of one q/k head, and in pass 1
    // also the S and M runs of one segment - form a group.  Workgroups are dealt to the 8 XCDs
    // round-robin by block index, so a group takes consecutive slots of ONE XCD: its members run at
    // the same time on CUs that share an L2, and the shared rows come from HBM once.
    const int G = HV / H;                         // value heads per q/k head
    const int64_t slot = blockIdx.x >> 3;
    const int xcd = blockIdx.x & 7;
    int64_t inh;
    int seg;
    int init = 0;                 // 0: from `src` (NULL = zero state), 1: identity, 2: zero
    int warm = 0;                 // chunks run before the segment proper, without output
    bool v_zero = false, src_user = false, dst_user = false;
    const float* src = nullptr;
    float* dst = nullptr;
    if (sp.kind == WIDE_WHOLE) {
        const int64_t group = (slot / G) * 8 + xcd;                 // (sequence, q/k head)
        if (group >= p.N * H) return;
        int64_t nseq = group / H;
        if (p.flags & GDN_FLAG_SEQ_ORDER) nseq = load_index(p.chunk_offsets, p.N + 1 + nseq, cu32);     // longest sequences start first
        inh = nseq * HV + (group % H) * G + slot % G; seg = 0;
        src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true;
        dst = p.ht ? p.ht + inh * (int64_t)(K * V) : nullptr; dst_user = true;
    } else if (sp.kind == WIDE_PASS1) {
        // group = (sequence, q/k head, segment 0 .. nseg-2); members: S runs of its value heads, then M runs
        const int64_t group = (slot / (2 * G)) * 8 + xcd;
        if (group >= p.N * H * (sp.nseg - 1)) return;
        const int member = (int)(slot % (2 * G));
        const int64_t nh = group / (sp.nseg - 1);
        seg = (int)(group % (sp.nseg - 1));
        inh = (nh / H) * HV + (nh % H) * G + member % G;
        // (a head whose segments all start warm needs no exact start states)
        if (sp.bound && !needs_exact_segments(sp, sp.bound + (inh / HV) * p.NT * HV + inh % HV, HV, lane)) return;
        if (member < G) {
            if (seg == 0) { src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true; }
            else init = 2;
            dst = sp.sloc + (inh * sp.nseg + seg) * 16384;
        } else {
            if (seg == 0) return;                                   // the first segment starts from the true state: no transition needed
            init = 1; v_zero = true;
            dst = sp.mseg + (inh * sp.nseg + seg) * 16384;
        }
    } else {
        const int64_t group = (slot / G) * 8 + xcd;                 // (sequence, q/k head, segment)
        if (group >= p.N * H * sp.nseg) return;
        const int64_t nh = group / sp.nseg;
        seg = (int)(group % sp.nseg);
        inh = (nh / H) * HV + (nh % H) * G + slot % G;
        if (seg == 0) { src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true; }
        else {
            // Warm start: begin `warm` chunks early from a zero state (from the true initial state when that reaches
            // the start of the sequence) and produce no output until the segment proper.  Heads with a segment that
            // cannot be started this way take the exact start states of the first pass and the merge.
            const float* bnd = sp.bound ? sp.bound + (inh / HV) * p.NT * HV + inh % HV : nullptr;
            int wch = 0;
            if (bnd && !needs_exact_segments(sp, bnd, HV, lane, seg, &wch)) {
                warm = __builtin_amdgcn_readfirstlane(wch);
                if ((int64_t)seg * sp.seg_chunks - warm == 0) { src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true; }
                else init = 2;
            } else {
                src = sp.sin + (inh * sp.nseg + seg) * 16384;
            }
        }
        if (seg == sp.nseg - 1 && p.ht) { dst = p.ht + inh * (int64_t)(K * V); dst_user = true; }
    }
    const int64_t n = inh / HV;
    const int hv = (int)(inh % HV);
    const int h = hv / (HV / H);

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
    const int64_t it0 = (int64_t)seg * sp.seg_chunks - warm;
    const int64_t it1 = min(nt, (int64_t)seg * sp.seg_chunks + sp.seg_chunks);
    const int64_t nsteps = it1 - it0;                       // may be <= 0 for an empty sequence
    const int64_t lastc = it1 - 1;
    char* otile = smem + KBUF + 3 * 16384;                  // [64 token rows][OT_PITCH]
    // The copy waves form P of a chunk while the compute waves are busy with the first products of its step and
    // announce it by adding to this counter (4 per step); a compute wave looks at the counter before it fetches P.
    // No barrier: one in the middle of a step costs the compute waves the slack between them.
    volatile int* pcount = (volatile int*)(smem + PCOUNT_OFF);
    if (tid == 0) *pcount = 0;                              // (published by the barrier B0)

    // =====================================================================================
    // Copy waves.  Step i (chunk it = it0 + i, stage cur = i & 1) has two phases, separated by
    // the workgroup barriers B1 (after the first half) and B2 (after the second half):
    //   phase A  compute waves read everything of stage cur and write the output tile
    //   phase B  compute waves read k of stage cur (transposed)
    // so the q / v / record part of a stage is free from B1 on and a k buffer from B2 on; all of
    // chunk it+1 must have landed at B2.  Loads complete in issue order, so "at most
    // N operations outstanding" proves that all but the N newest have landed.
    // =====================================================================================
    if (K < 128 && nsteps > 0) {
        // key features past K: clear the q and k tiles once; the copies never touch those pieces
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int i = tid; i < (2 * 16384) / 16; i += WIDE_THREADS) {
            *(u32x4*)(smem + (i >> 10) * STG_BYTES + STG_Q + (i & 1023) * 16) = z;
        }
        for (int i = tid; i < (3 * 16384) / 16; i += WIDE_THREADS) *(u32x4*)(smem + KBUF + i * 16) = z;
        lds_barrier();
    }
    if (w >= CW) {
        if (nsteps <= 0) return;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
        // ---- P = scale tril(q k^T 2^(G_t - G_t')) of a chunk, formed here from the q and k tiles of its stage while
        // the compute waves multiply by the state: the four copy waves share the 10 non-zero 16 x 16 tiles (tile
        // (tt, tj): query tokens of t-tile tt, key tokens of tile tj <= tt), as the transposed product so that a result
        // is spread over the lanes exactly like the operand fragment the compute waves read.  A counter in LDS announces it
        // (announce_P). ----
        auto produce_P = [&](const char* st, const char* kbuf) {
            if constexpr (FULL) {
                __builtin_amdgcn_s_setprio(3);
                const int pw = w - CW;
                const V8* sK = (const V8*)kbuf;
                const V8* sQ = (const V8*)(st + STG_Q);
                const float* t2 = (const float*)(st + STG_TAB2);
                const int a_off = (c16 >> 2) * 64 + 4 * (c16 & 3) + ((g + (c16 >> 2)) & 3);
                auto frag = [&](int tt, int sp) {
                    V8 qb[KS];
#pragma unroll
                    for (int s4 = 0; s4 < KS; ++s4) qb[s4] = sQ[tt * 256 + 16 * s4 + a_off];
                    const int t = 16 * tt + c16;
                    float gt = t2[TAB2_G + t], st_ = t2[TAB2_NQS + t];
                    if (l2q) {                        // q is normalised here: P, and the table that scales the (q S) rows
                        const float nq = row_rnorm<T>(qb, c16);
                        st_ *= nq;
                        if (sp == 0 && g == 0) ((float*)(st + STG_TAB))[TAB_SG + t] *= nq;
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
                        for (int s4 = 0; s4 < KS; ++s4) acc = Mma<T>::run(sK[tj * 256 + 16 * s4 + a_off], qb[s4], acc);
                        const f32x4 gj = *(const f32x4*)(t2 + TAB2_G + 16 * tj + 4 * g), nj = *(const f32x4*)(t2 + TAB2_NK + 16 * tj + 4 * g);
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int j = 16 * tj + 4 * g + r;
                            // select, never multiply by a mask: 2^(G_t - G_j) may overflow above the diagonal
                            out[half * 4 + r] = from_f32<T>((t >= j) ? st_ * nj[r] * acc[r] * fast_exp2(gt - gj[r]) : 0.f);
                        }
                    }
                    store_frag<T>((char*)st + STG_P, tt, sp, lane, out);
                };
                if (pw == 0) frag(3, 0);
                else if (pw == 1) frag(3, 1);
                else if (pw == 2) { frag(2, 0); frag(0, 0); }
                else { frag(1, 0); frag(2, 1); }
            }
        };
        // ... and announces it: this wave's fragments of step i are in LDS (its LDS operations complete in order)
        auto announce_P = [&]() {
            if constexpr (FULL) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (lane == 0) __hip_atomic_fetch_add((int*)pcount, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __builtin_amdgcn_s_setprio(0);
            }
        };
        // Block gather: rows 4j .. 4j+3 of a [token][head][128] tensor.  Rows past the end of the
        // sequence re-read its last row: whatever they hold is finite and is multiplied by the zero
        // columns of Xb, the zero rows of v_new and the causal zeros of P.
        // A copy wave moves one tensor: k (wave CW), q (CW+1) or v (CW+2), whose rows hold `dim` = K or V elements
        // (a multiple of 8, <= 128).  Pieces of q and k past K stay zero in LDS (the tiles were cleared once and those
        // lanes copy nothing); pieces of v past V re-read valid ones: value columns never mix, and the padded ones
        // are never stored.  What a lane fetches depends on the block only through j % 4: prepared once.
        const bool is_v = (w == CW + 2);
        const int dim = is_v ? V : K, pieces = dim >> 3;
        const int heads = is_v ? HV : H, head = is_v ? hv : h;
        const uint32_t row_bytes = (uint32_t)(heads * dim * 2);
        uint32_t piece_off[4];
        uint64_t piece_mask[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int c = 4 * g + ((c16 - jj) & 3);                         // this lane's slot holds piece c of row 4j + r
            piece_off[jj] = 16 * (is_v ? c % pieces : c);
            piece_mask[jj] = __builtin_amdgcn_ballot_w64(is_v || c < pieces);
        }
        // `skip`: the copy is issued with no lane enabled (nothing moves, the count of operations in flight is the same):
        // for what only the output needs (q, P) in the chunks of a warm-up, whose output nobody wants.
        auto gather_blocks = [&](const T* tensor, int64_t it, int j0, int j1, uint32_t lds_tile, bool skip = false) {
            const int64_t tok0 = bos + it * CH;
            const int valid = (int)min((int64_t)CH, len - it * CH);
            const char* base = (const char*)(tensor + (tok0 * heads + head) * dim);
            const uint32_t keep32 = __builtin_amdgcn_readfirstlane(skip ? 0u : ~0u);      // (scalar registers, never a literal)
            const uint64_t keep = ((uint64_t)keep32 << 32) | keep32;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                if (j < j0 || j >= j1) continue;
                const int row = min(4 * j + (c16 >> 2), valid - 1);
                const uint32_t voff = (uint32_t)row * row_bytes + piece_off[j & 3];
                if constexpr (DIMS128) {
                    if (FULL && warm > 0) gather_1k_to_lds_masked(base, voff, lds_tile + j * 1024, keep);
                    else gather_1k_to_lds(base, voff, lds_tile + j * 1024);
                } else {
                    gather_1k_to_lds_masked(base, voff, lds_tile + j * 1024, piece_mask[j & 3] & keep);
                }
            }
        };
        auto copy_rec = [&](int64_t it, int from, int to, uint32_t lds_stage, bool skip = false) {
            const char* rec = p.ws.Rec + ((boh + it) * HV + hv) * REC_BYTES;
            const uint32_t keep32 = __builtin_amdgcn_readfirstlane(skip ? 0u : ~0u);
            const uint64_t keep = ((uint64_t)keep32 << 32) | keep32;
#pragma unroll
            for (int j = 0; j < (int)(REC_BYTES / 1024); ++j)
                if (j >= from && j < to) {
                    if (FULL && warm > 0) gather_1k_to_lds_masked(rec + j * 1024, lane * 16, lds_stage + STG_REC + j * 1024, keep);
                    else gather_1k_to_lds(rec + j * 1024, lane * 16, lds_stage + STG_REC + j * 1024);
                }
        };
        if (w == CW) {
            // ---- k: the copy of chunk i+2 is issued at the start of step i (its buffer was last read
            // in step i-1) and awaited at the end of step i+1 ----
            auto issue_k = [&](int64_t i) {                                 // i counts from the first chunk of this run
                gather_blocks((const T*)p.k, min(it0 + i, lastc), 0, 16, lds0 + KBUF + (int)(i % 3) * 16384);
            };
            issue_k(0);
            issue_k(1);
            wait_vm_at_most<16>();
            lds_barrier();                                                  // B0: chunk 0 is complete
            for (int64_t i = 0; i < nsteps; ++i) {
                if (i >= warm) produce_P(smem + (i & 1) * STG_BYTES, smem + KBUF + (int)(i % 3) * 16384);
                announce_P();
                issue_k(i + 2);
                lds_barrier();                                              // B1
                wait_vm_at_most<16>();                                      // all but the newest copy: chunk i+1 has landed
                lds_barrier();                                              // B2
            }
        } else if (w <= CW + 2) {
            // ---- q + Xb + tables (wave CW+1) and v (wave CW+2).  Pieces
            // [0, XB) of chunk c are issued in phase B of step c-2, the rest in phase A of step c-1.
            const bool qside = (w == CW + 1);
            constexpr int XB = 8;
            auto issue = [&](int64_t it, int stage, bool early) {
                const uint32_t st = lds0 + stage * STG_BYTES;
                const bool warming = it - it0 < warm;               // a chunk of the warm-up: no output, so neither q nor P
                if (qside) {
                    if constexpr (FULL) {
                        // 16 q pieces, then Xb (5) and the tables (2)
                        if (early) gather_blocks((const T*)p.q, it, 0, 8, st + STG_Q, warming);
                        else { gather_blocks((const T*)p.q, it, 8, 16, st + STG_Q, warming); copy_rec(it, 0, REC_PIECES_X, st); copy_rec(it, REC_PIECE_TAB, REC_PIECE_TAB + 1, st); copy_rec(it, REC_PIECE_TAB2, REC_PIECE_TAB2 + 1, st, warming); }
                    } else {
                        if (early) { copy_rec(it, 0, REC_PIECES_X, st); copy_rec(it, REC_PIECE_TAB, REC_PIECE_TAB + 1, st); }      // all 6 pieces
                    }
                } else {
                    if (early) { if (!v_zero) gather_blocks((const T*)p.v, it, 0, 8, st + STG_V); }      // (v is not read when it counts as zero)
                    else {
                        if (!v_zero) gather_blocks((const T*)p.v, it, 8, 16, st + STG_V);
                    }
                }
            };
            // number of pieces issued early: 8, except 6 for the q side of a state-only run
            auto wait_early_only = [&]() {
                if (!FULL && qside) wait_vm_at_most<REC_PIECES_X + 1>();
                else wait_vm_at_most<XB>();
            };
            issue(it0, 0, true);
            issue(it0, 0, false);
            issue(min(it0 + 1, lastc), 1, true);
            wait_early_only();
            lds_barrier();                                                  // B0
            for (int64_t i = 0; i < nsteps; ++i) {
                const int64_t it = it0 + i;
                const int cur = (int)(i & 1);
                if (i >= warm) produce_P(smem + cur * STG_BYTES, smem + KBUF + (int)(i % 3) * 16384);
                announce_P();
                issue(min(it + 1, lastc), cur ^ 1, false);
                lds_barrier();                                              // B1
                issue(min(it + 2, lastc), cur, true);
                wait_early_only();                                          // chunk it+1 is complete
                lds_barrier();                                              // B2
            }
        } else {
            // ---- output rows: one instruction stores 4 token rows of 256 bytes ----
            T* og = (T*)p.o;
            u32x4 orow[16];                                                 // output tile of the previous chunk
            auto store_rows = [&](int64_t it) {
                const int valid = (int)min((int64_t)CH, len - it * CH);
                int64_t stride = (int64_t)HV * V * 4;                     // elements between rows 4 apart
                asm volatile("" : "+s"(stride));                            // keep the 16 row addresses out of long-lived registers
                T* dstp = og + ((bos + it * CH + g) * HV + hv) * V + c16 * 8;
                const bool col_ok = c16 * 8 < V;                          // (value columns past V exist in the tile only)
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    if (4 * j + g < valid && col_ok) *(u32x4*)dstp = orow[j];
                    dstp += stride;
                }
            };
            lds_barrier();                                                  // B0
            for (int64_t i = 0; i < nsteps; ++i) {
                if (i >= warm) produce_P(smem + (i & 1) * STG_BYTES, smem + KBUF + (int)(i % 3) * 16384);
                announce_P();
                if constexpr (FULL) { if (i > warm) store_rows(it0 + i - 1); }
                lds_barrier();                                              // B1
                if constexpr (FULL) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) orow[j] = *(const u32x4*)(otile + (4 * j + g) * OT_PITCH + c16 * 16);
                }
                lds_barrier();                                              // B2 (waits for the tile reads)
            }
            if constexpr (FULL) { if (nsteps > warm) store_rows(lastc); }
        }
        wait_vm_at_most<0>();                               // no copy may land in LDS after this workgroup has gone
        return;
    }

    // =====================================================================================
    // Compute waves
    // =====================================================================================
    // ---- state: all key rows (permuted, see above), value columns 16w .. 16w+15, C/D layout ----
    constexpr int NN = SMALL ? 1 : WIDE_NN;           // 16-column tiles per compute wave
    f32x4 S[2 * KS][NN];
#pragma unroll
    for (int m = 0; m < 2 * KS; ++m)
#pragma unroll
    for (int nn = 0; nn < NN; ++nn) {
        const int kk = 32 * (m >> 1) + 8 * g + 4 * (m & 1), vc = 16 * (NN * w + nn) + c16;
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

    // Lazy decay: the registers hold Shat = S / Gamma with one scalar Gamma = 2^lg per workgroup,
    // so the decay of the whole state by 2^G_last per chunk costs nothing: products with S are
    // rescaled by Gamma (folded into multiplies that exist anyway) and the update is divided by
    // the new Gamma (folded into the decay factors of v_new).  When Gamma gets small the state
    // is rescaled once and Gamma restarts at 1.  f16 operands have too little range for Shat, so
    // there the state is rescaled on every chunk.
    constexpr float LG_MIN = std::is_same<T, bf16_t>::value ? -60.f : 1.f;
    float lg = 0.f;

    // element offsets of this lane's LDS reads.  A transpose read hands lane 4j+e element e of the
    // four 4-element runs addressed by lanes j, j+4, j+8, j+12 of its 16-lane group: this lane
    // addresses row i = c16/4 of the 4-row run and column group j = c16%4.
    const int tr_i = c16 >> 2, tr_j = c16 & 3;
    const int a_off = (c16 >> 2) * 64 + 4 * (c16 & 3) + ((g + (c16 >> 2)) & 3);  // operand piece 4s + g of row c16 of a t-tile: + tt*256 + 16*s  (16-byte units)
    const int k_tr = (g * 64 + 4 * tr_i + ((tr_j + g) & 3)) * 8;                 // row 4g+i of a 16-row group, piece 4*(m/2) + j: + (32*sp2 + 16*half)*128 + 128*(m/2) + 4*(m&1)  (elements)
    int v_tr[NN];                                                                 // row 4g+i, piece = 8-column group of tile nn: + tt*2048
#pragma unroll
    for (int nn = 0; nn < NN; ++nn) {
        const int c = 2 * (NN * w + nn) + (tr_j >> 1);
        v_tr[nn] = (g * 64 + 16 * (c >> 2) + 4 * tr_i + ((c + g) & 3)) * 8 + 4 * (tr_j & 1);
    }

    // One step, written as a fixed sequence of small scheduling regions (the compiler may reorder
    // inside a region, not across `fence`).  A lone wave per SIMD has nobody to hide LDS latency
    // behind, so every LDS read is issued two or more regions before its first use (a rolling
    // window of three operand fragments), and the thin, dependent part of a step (D -> v_new ->
    // output of a pair of t-tiles) is cut into pieces that each share a region with four
    // independent matrix instructions (products of the next tiles, or the state update).
    auto step = [&](const char* st, const char* kbuf, int p_target) {
        const V8* sK = (const V8*)kbuf;
        const V8* sQ = (const V8*)(st + STG_Q);
        const T* sV = (const T*)(st + STG_V);
        const T* sKt = (const T*)kbuf;
        const char* sX = st + STG_X;
        const char* sP = st + STG_P;
        const float* sTab = (const float*)(st + STG_TAB);
        auto fence = [] { __builtin_amdgcn_sched_barrier(0); };

        // fragment f = (t-tile f/4, key tiles (2s, 2s+1) with s = f%4) of k and q, in a ring of RING register sets
        constexpr int RING = WIDE_RING;
        V8 ak[RING], aq[RING];
        auto F = [&](int f) {
            ak[f % RING] = sK[(f / KS) * 256 + 16 * (f % KS) + a_off];
            if constexpr (FULL) aq[f % RING] = sQ[(f / KS) * 256 + 16 * (f % KS) + a_off];
        };
        f32x4 ks[4][NN], ao[4][NN];
        V8 Sb[KS][NN];
        auto M = [&](int f) {                   // (k S) and (q S)^T contributions of fragment f
            const int tt = f / KS, sx = f % KS;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) {
                ks[tt][nn] = Mma<T>::run(ak[f % RING], Sb[sx][nn], sx ? ks[tt][nn] : f32x4{0.f, 0.f, 0.f, 0.f});
                if constexpr (FULL) ao[tt][nn] = Mma<T>::run(Sb[sx][nn], aq[f % RING], sx ? ao[tt][nn] : f32x4{0.f, 0.f, 0.f, 0.f});
            }
        };
        V4 vv[4][NN];                           // v in C/D layout, per t-tile
        V8 ax[4][2], ap[4][2];                  // Xb and P fragments [t-tile][column pair]
        auto FV = [&](int tt) {
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) vv[tt][nn] = Mma<T>::tr_read(sV + tt * 2048 + v_tr[nn]);
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
        V8 kt[2][2 * KS];                       // k^T rows of key tile m over t-tile pair sp2
        auto FK = [&](int sp2, int m) {
            const T* a = sKt + sp2 * 4096 + 128 * (m >> 1) + 4 * (m & 1) + k_tr;
            kt[sp2][m] = join<V8>(Mma<T>::tr_read(a), Mma<T>::tr_read(a + 2048));
        };
        float gamma, vscale;
        V8 Db[2][NN], Vn[2][NN], Vg[2][NN];
        auto TD = [&](int tt) {                 // D = v - 2^G (k S), rows of t-tile tt
            const f32x4 eg = *(const f32x4*)(sTab + TAB_EG + 16 * tt + 4 * g) * gamma;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float x = (!FULL && v_zero) ? 0.f : to_f32(vv[tt][nn][r]);      // (full runs always have their v)
                    Db[tt >> 1][nn][(tt & 1) * 4 + r] = from_f32<T>(x - eg[r] * ks[tt][nn][r]);
                }
        };
        // The matrix part and the conversion of its result sit in different regions: a vector
        // instruction that needs the result of a matrix instruction issued just before it stalls
        // for the whole latency of the matrix pipeline.
        f32x4 vn[4][NN], oacc[4][NN];
        auto TXa = [&](int tt) {                // v_new = Xb D (lower triangular)
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) {
                vn[tt][nn] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int sp2 = 0; sp2 <= (tt >> 1); ++sp2) vn[tt][nn] = Mma<T>::run(ax[tt][sp2], Db[sp2][nn], vn[tt][nn]);
            }
        };
        auto TXb = [&](int tt) {                // ... as B operands: plain, and decayed to the chunk end
            const f32x4 dec = *(const f32x4*)(sTab + TAB_DEC + 16 * tt + 4 * g) * vscale;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    Vn[tt >> 1][nn][(tt & 1) * 4 + r] = from_f32<T>(vn[tt][nn][r]);
                    Vg[tt >> 1][nn][(tt & 1) * 4 + r] = from_f32<T>(vn[tt][nn][r] * dec[r]);
                }
        };
        auto TPa = [&](int tt) {                // o^T = scale 2^G (q S)^T + (P v_new)^T
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
        auto TPb = [&](int tt) {                // ... to the output tile: 4 consecutive value columns of a token row per lane
            if constexpr (FULL) {
#pragma unroll
                for (int nn = 0; nn < NN; ++nn) {
                    V4 o4;
#pragma unroll
                    for (int r = 0; r < 4; ++r) o4[r] = from_f32<T>(oacc[tt][nn][r]);
                    *(V4*)(otile + (16 * tt + c16) * OT_PITCH + (16 * (NN * w + nn) + 4 * g) * 2) = o4;
                }
            }
        };
        auto U = [&](int sp2, int m) {          // S += k^T (v_new decayed): key tile m, t-tile pair sp2
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) S[m][nn] = Mma<T>::run(kt[sp2][m], Vg[sp2][nn], S[m][nn]);
        };

        // ---- the state as B operand (pairs of key tiles (2s, 2s+1) = key features 32s + 8g + e) ----
#pragma unroll
        for (int f = 0; f < RING - 1; ++f) F(f);
#pragma unroll
        for (int s = 0; s < KS; ++s)
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
        auto wait_P = [&]() {
            // P of this chunk: normally long there (the copy waves form it first thing in a step, at raised priority)
            if constexpr (FULL) { while (*pcount < p_target) __builtin_amdgcn_s_sleep(1); }
        };
        auto fold = [&]() {                     // the decay fold: rare, a scalar branch so that it is not if-converted into the common path
            if (__builtin_amdgcn_readfirstlane((int)lazy) == 0) {
                const float fo = fast_exp2(lg_try);
#pragma unroll
                for (int m = 0; m < 2 * KS; ++m)
#pragma unroll
                    for (int nn = 0; nn < NN; ++nn) S[m][nn] *= fo;
            }
            lg = lazy ? lg_try : 0.f;
        };
        if constexpr (SMALL) {
            // ---- eight fragments (two per t-tile), four state tiles per wave.  The chain that the next step waits for
            // is M(7) -> D, v_new of t-tiles 2, 3 -> their state update; the tail of tiles 0, 1 and everything of the
            // output fill its gaps ----
            F(2); M(0); FV(0); FV(1); fence();
            F(3); M(1); FX(0); FX(1); fence();
            F(4); M(2); FV(2); FV(3); fence();
            F(5); M(3); FX(2); FX(3); fence();
            F(6); M(4); TD(0); TD(1); FK(0, 0); FK(0, 1); fence();
            F(7); M(5); TXa(0); TXa(1); FK(0, 2); FK(0, 3); fence();
            M(6); TXb(0); TXb(1); FK(1, 0); FK(1, 1); fence();
            M(7); FK(1, 2); FK(1, 3); fence();
            fold();
            TD(2); TD(3); U(0, 0); U(0, 1); U(0, 2); U(0, 3); fence();
            TXa(2); TXa(3); wait_P(); FP(0); FP(1); FP(2); FP(3); fence();
            TXb(2); TXb(3); TPa(0); TPa(1); fence();
            U(1, 0); U(1, 1); TPb(0); TPb(1); TPa(2); TPa(3); fence();
            TPb(2); TPb(3); fence();
            lds_barrier();                                          // B1
            U(1, 2); U(1, 3); fence();
            lds_barrier();                                          // B2
        } else {
            // ---- sixteen regions: the products of fragment f, the fetch of fragment f + RING - 1, and beside them
            // the other fetches (t-tiles 0, 1) and then the tail of tiles 0, 1 while tiles 2, 3 are multiplied ----
    #pragma unroll
            for (int f = 0; f < 16; ++f) {
                if (f + RING - 1 < 16) F(f + RING - 1);
                M(f);
                if (f == 4) FV(0);
                if (f == 5) FV(1);
                if (f == 6) FX(0);
                if (f == 7) FX(1);
                if (f == 8) TD(0);
                if (f == 9) { TD(1); }
                if (f == 10) { TXa(0); TXa(1); }
                if (f == 11) {
                    wait_P();
                    FP(0); FP(1);
                }
                if (f == 11) { TXb(0); TXb(1); FV(2); }
                if (f == 12) { TPa(0); TPa(1); FV(3); }
                if (f == 13) { TPb(0); TPb(1); FX(2); }
                if (f == 14) { FX(3); FK(0, 0); FK(0, 1); }
                if (f == 15) { FK(0, 2); FK(0, 3); }
                fence();
            }
            fold();
            // ---- state update from tiles 0, 1, with the tail of tiles 2, 3 ----
            U(0, 0); U(0, 1); TD(2); FK(0, 4); FK(0, 5); fence();
            U(0, 2); U(0, 3); TD(3); FK(0, 6); FK(0, 7); FP(2); fence();
            U(0, 4); U(0, 5); TXa(2); TXa(3); FK(1, 0); FK(1, 1); FP(3); fence();
            U(0, 6); U(0, 7); TXb(2); TXb(3); FK(1, 2); FK(1, 3); fence();
            // ... and the first half of the update from tiles 2, 3
            U(1, 0); U(1, 1); TPa(2); TPa(3); FK(1, 4); FK(1, 5); fence();
            U(1, 2); U(1, 3); TPb(2); TPb(3); FK(1, 6); FK(1, 7); fence();
            lds_barrier();                                          // B1: q, v, record of this stage are free
            // ---- rest of the state update from tiles 2, 3 ----
    #pragma unroll
            for (int m = 4; m < 8; ++m) U(1, m);
            fence();
            lds_barrier();                                          // B2: k of this stage is free, the other stage is complete
        }
    };
    if (nsteps > 0) {
        lds_barrier();                                          // B0: the copy waves have filled stage 0
        for (int64_t i = 0; i < nsteps; ++i) {
            step(smem + (i & 1) * STG_BYTES, smem + KBUF + (int)(i % 3) * 16384, 4 * ((int)i + 1));
        }
    }

    if (dst) {
        if constexpr (SMALL) {
            // the buffers of the segment passes are [128][128] and the merge reads all of them: zero what this state leaves out
            if (!dst_user) {
                for (int i = tid; i < 4096; i += CW * 64) {
                    const int row = i >> 5, c4 = (i & 31) * 4;
                    if (row >= 64 || c4 >= 64) *(f32x4*)(dst + row * 128 + c4) = f32x4{0.f, 0.f, 0.f, 0.f};
                }
            }
        }
        const float gamma = fast_exp2(lg);
#pragma unroll
        for (int m = 0; m < 2 * KS; ++m)
#pragma unroll
        for (int nn = 0; nn < NN; ++nn) {
            const int kk = 32 * (m >> 1) + 8 * g + 4 * (m & 1), vc = 16 * (NN * w + nn) + c16;
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

// S_in[j+1] = M_j S_in[j] + S_loc,j for j = 1 .. nseg-2, with S_in[1] = S_loc,0 (the run of segment 0
// started from the true initial state).  fp32 throughout (fp32 matrix cores): one workgroup per
// (sequence, head, slab of 16 value columns); M_j is staged in LDS, the next one travels in registers
// meanwhile (fetched with consecutive lanes on consecutive addresses: read straight into the operand
// registers, where neighbouring lanes hold different rows, the same bytes take longer).  The 8 slabs
// of a head sit on one XCD (block index mod 8), so that M_j comes from HBM once.
// Contraction indices of the 16x16x4 products: step e of block q uses {16q + 4g + e}, so a lane
// reads its four values of A (a row of M) and of B (a column of S, kept transposed) as one 16-byte
// LDS read each.
constexpr int MP = 132;                            // pitch of the staged rows (floats): conflict-free 16-byte reads
constexpr size_t MERGE_SMEM = (128 * MP + 16 * MP) * 4;

__global__ __launch_bounds__(256) void gdn_segment_merge_kernel(SegmentPlan sp, int64_t NH, int HV, int64_t NT) {
    extern __shared__ __align__(16) char smem[];
    float* sM = (float*)smem;                      // [128 i][MP] M_j
    float* sSt = sM + 128 * MP;                    // [16 n][MP] current S_in slab, transposed
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    const int64_t inh = (int64_t)(blockIdx.x >> 6) * 8 + (blockIdx.x & 7);
    if (inh >= NH) return;
    if (sp.bound && !needs_exact_segments(sp, sp.bound + (inh / HV) * NT * HV + inh % HV, HV, lane)) return;      // all segments start warm
    const int v0 = (int)((blockIdx.x >> 3) & 7) * 16;
    const int nseg = sp.nseg;
    f32x4 pre[16];
    auto fetch_M = [&](int j) {
        const float* M = sp.mseg + (inh * nseg + j) * 16384;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int idx = tid + 256 * i;
            pre[i] = *(const f32x4*)(M + (idx >> 5) * 128 + (idx & 31) * 4);
        }
    };
    if (nseg > 2) fetch_M(1);
    // this wave's part of a slab: key tiles 2w, 2w+1 in C/D layout (column c16, rows 4g .. 4g+3)
    auto slab_rows = [&](const float* base, int j, f32x4 (&x)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) x[i][r] = base[(inh * nseg + j) * 16384 + (16 * (2 * w + i) + 4 * g + r) * 128 + v0 + c16];
    };
    auto publish = [&](int j, const f32x4 (&x)[2]) {          // x becomes S_in[j]: to the other waves (transposed) and to memory
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *(f32x4*)(sSt + c16 * MP + 16 * (2 * w + i) + 4 * g) = x[i];
#pragma unroll
            for (int r = 0; r < 4; ++r) sp.sin[(inh * nseg + j) * 16384 + (16 * (2 * w + i) + 4 * g + r) * 128 + v0 + c16] = x[i][r];
        }
    };
    f32x4 x[2];
    slab_rows(sp.sloc, 0, x);
    publish(1, x);
    for (int j = 1; j + 1 < nseg; ++j) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int idx = tid + 256 * i;
            *(f32x4*)(sM + (idx >> 5) * MP + (idx & 31) * 4) = pre[i];
        }
        if (j + 2 < nseg) fetch_M(j + 1);
        f32x4 sl[2];
        slab_rows(sp.sloc, j, sl);
        __syncthreads();                            // M_j and S_in[j] are complete
        f32x4 acc[2][2];                            // two accumulation chains per tile (even / odd blocks)
#pragma unroll
        for (int i = 0; i < 2; ++i) acc[i][0] = acc[i][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const f32x4 b = *(const f32x4*)(sSt + c16 * MP + 16 * q + 4 * g);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const f32x4 a = *(const f32x4*)(sM + (16 * (2 * w + i) + c16) * MP + 16 * q + 4 * g);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][q & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], acc[i][q & 1], 0, 0, 0);
            }
        }
        __syncthreads();                            // all waves have read M_j and S_in[j]
#pragma unroll
        for (int i = 0; i < 2; ++i) x[i] = acc[i][0] + acc[i][1] + sl[i];
        publish(j + 1, x);
    }
}

template <typename T, bool FULL, bool DIMS128, bool SMALL>
static int launch_wide_dims(const ChunkParams& p, const SegmentPlan& sp, int64_t blocks, hipStream_t stream) {
    auto kern = gdn_chunk_wide_kernel<T, FULL, DIMS128, SMALL>;
    static SmemAttrDone attr_done;       // per instantiation
    if (int rc = ensure_dynamic_smem((const void*)kern, WIDE_SMEM, attr_done, "hipFuncSetAttribute(wide)")) return rc;
    if (blocks <= 0) return GDN_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(WIDE_THREADS), WIDE_SMEM, stream, p, sp);
    return check_launch("gdn_chunk_wide_kernel");
}

template <typename T, bool FULL>
static int launch_wide_kind(const ChunkParams& p, const SegmentPlan& sp, int64_t blocks, hipStream_t stream) {
    if (p.K == 128 && p.V == 128) return launch_wide_dims<T, FULL, true, false>(p, sp, blocks, stream);
    if (p.K <= 64 && p.V <= 64) return launch_wide_dims<T, FULL, false, true>(p, sp, blocks, stream);
    return launch_wide_dims<T, FULL, false, false>(p, sp, blocks, stream);
}

// sp.kind selects the work (whole sequences, pass 1 or pass 2 of the segment-parallel evaluation)
template <typename T>
int launch_wide(const ChunkParams& p, SegmentPlan sp, hipStream_t stream) {
    const int64_t G = p.HV / p.H;
    if (sp.kind == WIDE_PASS1)
        return launch_wide_kind<T, false>(p, sp, (p.N * p.H * (sp.nseg - 1) + 7) / 8 * 8 * 2 * G, stream);
    if (sp.kind == WIDE_WHOLE) {
        sp.nseg = 1;
        sp.seg_chunks = 1 << 30;
        return launch_wide_kind<T, true>(p, sp, (p.N * p.H + 7) / 8 * 8 * G, stream);
    }
    return launch_wide_kind<T, true>(p, sp, (p.N * p.H * sp.nseg + 7) / 8 * 8 * G, stream);
}

int launch_segment_merge(const ChunkParams& p, SegmentPlan sp, hipStream_t stream) {
    static SmemAttrDone attr_done;
    if (int rc = ensure_dynamic_smem((const void*)gdn_segment_merge_kernel, MERGE_SMEM, attr_done, "hipFuncSetAttribute(merge)")) return rc;
    hipLaunchKernelGGL(gdn_segment_merge_kernel, dim3((unsigned)((p.NH + 7) / 8 * 64)), dim3(256), MERGE_SMEM, stream, sp, p.NH, p.HV, p.NT);
    return check_launch("gdn_segment_merge_kernel");
}

template int launch_wide<bf16_t>(const ChunkParams&, SegmentPlan, hipStream_t);
template int launch_wide<f16_t>(const ChunkParams&, SegmentPlan, hipStream_t);

}  // namespace gdn
