// Sequential stage of the chunked prefill for WIDE keys, 128 < K <= 256 (the reference's scan holds up to four
// [64, BV] state tiles, i.e. K <= 256: fla/ops/common/chunk_delta_h.py:108-114, 210-315).  Same step as
// gdn_chunk_wide.hip,
//   D = v - 2^G (k S),  v_new = Xb D,  o = scale 2^G (q S) + P v_new,  S = 2^G_last S + k^T (v_new 2^(G_last-G)),
// with the state of one workgroup cut along the VALUE columns instead: a workgroup owns 64 value columns of one
// (sequence, value head) for all 256 key rows (the value columns of the recurrence never mix), compute wave w the
// columns 16w .. 16w+15: 16 state tiles of 16 x 16 per wave, the same 64 registers as the 128 x 32 slab of the
// narrow kernel.  A head with V value columns takes ceil(V / 64) workgroups, which share the head's record and, with
// the other value heads of the q/k head, its k and q rows (consecutive slots of one XCD: one L2).
//
// k and q tiles are two 128-feature halves, each laid out exactly like the narrow kernel's tile, so every operand
// address is the narrow kernel's plus a half offset.  What differs is the LDS budget: 64 tokens x 512 B of k and of
// q are 32 KB each.  k has two buffers (read until the very end of a step, copied one step ahead), v and the record
// have two, q and P have ONE: q of the next chunk is requested after the barrier that ends this chunk's last read of
// it and awaited in the middle of the next step - a step multiplies by k first (the products that head the chain to the
// next state) and turns to q, P and the output when an LDS counter says that q has landed.
//
// Long dense sequences on few heads are cut into time segments.  A segment starts warm where the decay allows it (see
// WARM_LOG2); a head with a segment that cannot start warm takes exact start states, S_out = M S_in + S_loc per segment as in
// gdn_chunk_wide.hip: pass 1 (FULL = false: no q, P, output) runs every segment but the last from zero (S_loc, 64 value
// columns per workgroup) and from the identity with v = 0 (the 256 x 256 transition M, 64 of its columns per
// workgroup), gdn_segment_merge256_kernel chains them in fp32, pass 2 starts every segment from its merged state.
#include "gdn_chunk_common.h"

namespace gdn {

constexpr int W2_KB = 0;                                  // two k buffers: [half][16 KB tile]
constexpr int W2_Q = 65536;                               // q: [half][16 KB tile]
constexpr int W2_V = 98304;                               // two v tiles, 64 rows of 256 B of which the first 128 B are used
constexpr int W2_REC = 131072;                            // two records without P
constexpr int W2_RX = 0, W2_RTAB = 5120, W2_RTAB2 = 6144, W2_REC_BYTES = 7168;
constexpr int W2_P = W2_REC + 2 * W2_REC_BYTES;           // P of the current chunk, formed here
constexpr int W2_OT = W2_P + 5120;                        // output tile [64 tokens][W2_OT_PITCH]
constexpr int W2_OT_PITCH = 144;                          // 128 B of a row + pad
constexpr int W2_PCOUNT = W2_OT + 64 * W2_OT_PITCH;
constexpr size_t W2_SMEM = W2_PCOUNT + 16;                // 159 760 B
constexpr int W2_CW = 4;                                  // compute waves
constexpr int W2_THREADS = (W2_CW + 4) * 64;

template <typename T, bool FULL>
__global__ __launch_bounds__(W2_THREADS) void gdn_chunk_wide256_kernel(ChunkParams p, int NVB, SegmentPlan sp) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    const int K = p.K, V = p.V;
    const int tid = threadIdx.x, lane = tid & 63, c16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int H = p.H, HV = p.HV;
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    const bool l2q = p.flags & FLAG_Q_NORM_IN_SCAN;       // q is l2-normalised where P is formed (row factors)
    const bool vfirst = p.flags & GDN_FLAG_STATE_V_FIRST;

    // ---- which (sequence, value head, block of value columns): the workgroups that read the same k and q rows take
    // consecutive slots of one XCD (block index mod 8) ----
    // Pass 1 (FULL = false) adds, per value head, four workgroups for the 64-column blocks of the transition M.
    const int G = HV / H, NMB = FULL ? 0 : W2_KD / W2_VB, GV = G * (NVB + NMB);
    const int VP = NVB * W2_VB;                                      // value columns of the segment buffers
    const int64_t slot = blockIdx.x >> 3;
    const int xcd = blockIdx.x & 7;
    const int64_t group = (slot / GV) * 8 + xcd;                     // (sequence, q/k head, time segment)
    const int nseg = sp.nseg;                                        // 1: whole sequences
    const int nrun = FULL ? nseg : nseg - 1;                         // (pass 1: every segment but the last)
    if (group >= p.N * H * nrun) return;
    const int seg = (int)(group % nrun);
    int64_t n = (group / nrun) / H;
    if (p.flags & GDN_FLAG_SEQ_ORDER) n = load_index(p.chunk_offsets, p.N + 1 + n, cu32);
    const int h = (int)((group / nrun) % H);
    const int member = (int)(slot % GV);
    const bool m_run = !FULL && member >= G * NVB;                   // a block of columns of the transition matrix
    const int hv = h * G + (m_run ? (member - G * NVB) / NMB : member / NVB);
    const int v0 = (m_run ? (member - G * NVB) % NMB : member % NVB) * W2_VB;
    const int64_t inh = n * HV + hv;
    // Time segments start warm: a zero state a few chunks early, where the bound on the chunks' transitions makes the true
    // state irrelevant (see WARM_LOG2), and no output until the segment proper.  A head with a segment that cannot start
    // this way takes the exact start states of the first pass and the merge.
    int warm = 0;
    bool exact = false;
    if (nseg > 1) {
        int wch = 0;
        exact = !sp.bound || needs_exact_segments(sp, sp.bound + n * p.NT * HV + hv, HV, lane, seg, &wch);
        if (!exact && seg > 0) warm = __builtin_amdgcn_readfirstlane(wch);
    }
    if (!FULL && (!exact || (m_run && seg == 0))) return;            // (the first segment starts from the true state: no transition needed)
    // where the state comes from and goes to: the caller's tensors ([K][V] or [V][K], K x V entries), or the segment
    // buffers ([256][VP], for M [256][256])
    const size_t seg_floats = seg256_floats(V);
    float* seg_base = nseg > 1 ? p.ws.Seg + (size_t)(inh * nseg + seg) * seg_floats : nullptr;
    const bool from_start = nseg == 1 || (int64_t)seg * sp.seg_chunks - warm == 0, to_end = nseg == 1 || seg == nseg - 1;
    const float* src = nullptr;
    float* dst = nullptr;
    int init = 0;                                                    // 0: from src (NULL: zero), 1: identity
    bool src_user = false, dst_user = false;
    if (FULL) {
        if (from_start) { src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true; }
        else if (exact) src = seg_base + (size_t)W2_KD * VP + (size_t)W2_KD * W2_KD;       // S_in of this segment
        if (to_end && p.ht) { dst = p.ht + inh * (int64_t)(K * V); dst_user = true; }
    } else if (m_run) {
        init = 1;
        dst = seg_base + (size_t)W2_KD * VP;                         // M of this segment
    } else {
        if (seg == 0) { src = p.h0 ? p.h0 + inh * (int64_t)(K * V) : nullptr; src_user = true; }
        dst = seg_base;                                              // S_loc of this segment
    }
    const bool v_zero = m_run;

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
    const int64_t it0 = nseg == 1 ? 0 : (int64_t)seg * sp.seg_chunks - warm;       // first chunk of this run (warm-up included)
    const int64_t it1 = nseg == 1 ? nt : min(nt, (int64_t)(seg + 1) * sp.seg_chunks);
    const int64_t nsteps = it1 - it0;                                               // step i works on chunk it0 + i
    const int64_t lastc = it1 - 1;
    char* otile = smem + W2_OT;
    volatile int* pcount = (volatile int*)(smem + W2_PCOUNT);           // copy waves whose share of P of step i is in LDS: 4 (i + 1)
    volatile int* qcount = pcount + 1;                                   // chunks whose q tile has landed
    if (tid == 0) { *pcount = 0; *qcount = 0; }
    // Key features past K and value columns past V are never copied: the tiles are cleared once.
    if (nsteps > 0) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int i = tid; i < W2_REC / 16; i += W2_THREADS) *(u32x4*)(smem + i * 16) = z;
    }
    lds_barrier();

    const int a_off = (c16 >> 2) * 64 + 4 * (c16 & 3) + ((g + (c16 >> 2)) & 3);   // operand piece 4s + g of row c16 of a t-tile (16-byte units)

    // =====================================================================================
    // Copy waves.  Step i reads stage i & 1 of k, v and the record; barrier B1 ends the reads of q, v, the record and
    // the writes of the output tile, barrier B2 the reads of k.
    // =====================================================================================
    if (w >= W2_CW) {
        if (nsteps <= 0) return;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
        // P = scale tril(q k^T 2^(G_t - G_t')) of a chunk from its q and k tiles (see gdn_chunk_wide.hip), contraction
        // over both halves of the key features
        auto produce_P = [&](const char* kbuf, const char* rec, int q_target) {
            if constexpr (!FULL) return;
            while (*qcount < q_target) __builtin_amdgcn_s_sleep(1);          // q of this chunk has landed
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_setprio(3);
            const int pw = w - W2_CW;
            const V8* sK = (const V8*)kbuf;
            const V8* sQ = (const V8*)(smem + W2_Q);
            const float* t2 = (const float*)(rec + W2_RTAB2);
            auto frag = [&](int tt, int sp) {
                V8 qb[8];
#pragma unroll
                for (int s8 = 0; s8 < 8; ++s8) qb[s8] = sQ[(s8 >> 2) * 1024 + tt * 256 + 16 * (s8 & 3) + a_off];
                const int t = 16 * tt + c16;
                float gt = t2[TAB2_G + t], st_ = t2[TAB2_NQS + t];
                if (l2q) {                        // q is normalised here: P, and the table that scales the (q S) rows
                    const float nq = row_rnorm<T>(qb, c16);
                    st_ *= nq;
                    if (sp == 0 && g == 0) ((float*)(rec + W2_RTAB))[TAB_SG + t] *= nq;
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
                    for (int s8 = 0; s8 < 8; ++s8) acc = Mma<T>::run(sK[(s8 >> 2) * 1024 + tj * 256 + 16 * (s8 & 3) + a_off], qb[s8], acc);
                    const f32x4 gj = *(const f32x4*)(t2 + TAB2_G + 16 * tj + 4 * g), nj = *(const f32x4*)(t2 + TAB2_NK + 16 * tj + 4 * g);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int j = 16 * tj + 4 * g + r;
                        out[half * 4 + r] = from_f32<T>((t >= j) ? st_ * nj[r] * acc[r] * fast_exp2(gt - gj[r]) : 0.f);
                    }
                }
                store_frag<T>(smem + W2_P, tt, sp, lane, out);
            };
            if (pw == 0) frag(3, 0);
            else if (pw == 1) frag(3, 1);
            else if (pw == 2) { frag(2, 0); frag(0, 0); }
            else { frag(1, 0); frag(2, 1); }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0) __hip_atomic_fetch_add((int*)pcount, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __builtin_amdgcn_s_setprio(0);
        };
        // Rows 4j .. 4j+3 of a [token][head][K] tensor, 128 features of them (`half`), into block j of a 16 KB tile:
        // lane (g, c16) holds piece c = 4g + ((c16 - j) & 3) of row 4j + c16 / 4.  Rows past the end of the sequence
        // re-read its last row (finite, and multiplied by zeros everywhere).
        auto gather_qk = [&](const T* tensor, int64_t it, uint32_t lds_tile) {
            const int valid = (int)min((int64_t)CH, len - it * CH);
            const char* base = (const char*)(tensor + ((bos + it * CH) * H + h) * K);
            const uint32_t row_bytes = (uint32_t)(H * K * 2);
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int c = 4 * g + ((c16 - j) & 3);
                    const uint64_t mask = __builtin_amdgcn_ballot_w64(128 * half + 8 * c < K);
                    const int row = min(4 * j + (c16 >> 2), valid - 1);
                    gather_1k_to_lds_masked(base, (uint32_t)row * row_bytes + 256 * half + 16 * c, lds_tile + half * 16384 + j * 1024, mask);
                }
        };
        auto copy_rec = [&](int64_t it, uint32_t lds_rec) {
            const char* rec = p.ws.Rec + ((boh + it) * HV + hv) * REC_BYTES;
#pragma unroll
            for (int j = 0; j < REC_PIECES_X; ++j) gather_1k_to_lds(rec + REC_X + j * 1024, lane * 16, lds_rec + W2_RX + j * 1024);
            gather_1k_to_lds(rec + REC_TAB, lane * 16, lds_rec + W2_RTAB);
            gather_1k_to_lds(rec + REC_TAB2, lane * 16, lds_rec + W2_RTAB2);
        };
        if (w == W2_CW) {
            // ---- k: chunk i+1 is copied during step i (its buffer was last read in step i-1) ----
            gather_qk((const T*)p.k, it0, lds0 + W2_KB);
            wait_vm_at_most<0>();
            lds_barrier();                                                  // B0
            for (int64_t i = 0; i < nsteps; ++i) {
                gather_qk((const T*)p.k, min(it0 + i + 1, lastc), lds0 + W2_KB + (int)((i + 1) & 1) * 32768);
                produce_P(smem + W2_KB + (int)(i & 1) * 32768, smem + W2_REC + (int)(i & 1) * W2_REC_BYTES, (int)i + 1);
                lds_barrier();                                              // B1
                wait_vm_at_most<0>();
                lds_barrier();                                              // B2
            }
        } else if (w == W2_CW + 1) {
            // ---- q (one buffer) and the record (two).  q of chunk i+1 is requested right after the barrier B1 of step i,
            // which ends the last read of q of chunk i, and is awaited inside step i+1: the compute waves multiply by k
            // first and turn to q, and the copy waves to P, only when the counter says that it has landed ----
            if constexpr (FULL) gather_qk((const T*)p.q, it0, lds0 + W2_Q);
            copy_rec(it0, lds0 + W2_REC);
            wait_vm_at_most<0>();
            lds_barrier();                                                  // B0
            for (int64_t i = 0; i < nsteps; ++i) {
                copy_rec(min(it0 + i + 1, lastc), lds0 + W2_REC + (int)((i + 1) & 1) * W2_REC_BYTES);      // 7 operations
                wait_vm_at_most<7>();                                       // everything older than these: q of chunk i
                if (FULL && lane == 0) __hip_atomic_fetch_add((int*)qcount, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                produce_P(smem + W2_KB + (int)(i & 1) * 32768, smem + W2_REC + (int)(i & 1) * W2_REC_BYTES, (int)i + 1);
                lds_barrier();                                              // B1
                wait_vm_at_most<0>();                                       // the record of chunk i+1
                if (FULL && i + 1 < nsteps) gather_qk((const T*)p.q, it0 + i + 1, lds0 + W2_Q);
                lds_barrier();                                              // B2
            }
        } else if (w == W2_CW + 2) {
            // ---- v: the 64 columns of this workgroup, 4 rows per copy (lanes g < 2 hold the 8 pieces of a row) ----
            auto gather_v = [&](int64_t it, uint32_t lds_tile) {
                const int valid = (int)min((int64_t)CH, len - it * CH);
                const char* base = (const char*)((const T*)p.v + ((bos + it * CH) * HV + hv) * V + v0);
                const uint32_t row_bytes = (uint32_t)(HV * V * 2);
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int c = 4 * g + ((c16 - j) & 3);
                    const uint64_t mask = __builtin_amdgcn_ballot_w64(c < 8 && v0 + 8 * c < V);
                    const int row = min(4 * j + (c16 >> 2), valid - 1);
                    gather_1k_to_lds_masked(base, (uint32_t)row * row_bytes + 16 * c, lds_tile + j * 1024, mask);
                }
            };
            if (!v_zero) gather_v(it0, lds0 + W2_V);                        // (v is not read where it counts as zero)
            wait_vm_at_most<0>();
            lds_barrier();                                                  // B0
            for (int64_t i = 0; i < nsteps; ++i) {
                if (!v_zero) gather_v(min(it0 + i + 1, lastc), lds0 + W2_V + (int)((i + 1) & 1) * 16384);
                produce_P(smem + W2_KB + (int)(i & 1) * 32768, smem + W2_REC + (int)(i & 1) * W2_REC_BYTES, (int)i + 1);
                lds_barrier();                                              // B1
                wait_vm_at_most<0>();
                lds_barrier();                                              // B2
            }
        } else {
            // ---- output rows: one instruction stores 8 token rows of 128 bytes ----
            T* og = (T*)p.o;
            u32x4 orow[8];
            const int orow_r = lane >> 3, opiece = lane & 7;
            auto store_rows = [&](int64_t it) {
                const int valid = (int)min((int64_t)CH, len - it * CH);
                const bool col_ok = v0 + 8 * opiece < V;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int row = 8 * j + orow_r;
                    if (row < valid && col_ok) *(u32x4*)(og + ((bos + it * CH + row) * HV + hv) * V + v0 + 8 * opiece) = orow[j];
                }
            };
            lds_barrier();                                                  // B0
            for (int64_t i = 0; i < nsteps; ++i) {
                produce_P(smem + W2_KB + (int)(i & 1) * 32768, smem + W2_REC + (int)(i & 1) * W2_REC_BYTES, (int)i + 1);
                if (FULL && i > warm) store_rows(it0 + i - 1);     // (the chunks of a warm-up leave no output)
                lds_barrier();                                              // B1
                if constexpr (FULL) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) orow[j] = *(const u32x4*)(otile + (8 * j + orow_r) * W2_OT_PITCH + opiece * 16);
                }
                lds_barrier();                                              // B2 (waits for the tile reads)
            }
            if (FULL && nsteps > warm) store_rows(lastc);
        }
        wait_vm_at_most<0>();                               // no copy may land in LDS after this workgroup has gone
        return;
    }

    // =====================================================================================
    // Compute waves
    // =====================================================================================
    // state tile m (0..15), row 4g + r: key feature 32 (m/2) + 8g + 4 (m%2) + r; column: value v0 + 16w + c16
    f32x4 S[16];
    const int vc = v0 + 16 * w + c16;
    // the caller's state is [K][V] or [V][K]; the buffers of the segment passes are [256][VP] (M: [256][256])
    const int buf_pitch = m_run ? W2_KD : VP;
#pragma unroll
    for (int m = 0; m < 16; ++m) {
        const int kk = 32 * (m >> 1) + 8 * g + 4 * (m & 1);
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        if (init == 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] = (kk + r == vc) ? 1.f : 0.f;
        } else if (src) {
            const int sk = src_user ? (vfirst ? 1 : V) : buf_pitch, sv = src_user ? (vfirst ? K : 1) : 1;
            if (kk < (src_user ? K : W2_KD) && vc < (src_user ? V : buf_pitch)) {
                const float* e = src + (int64_t)kk * sk + (int64_t)vc * sv;
                s = f32x4{e[0], e[sk], e[2 * sk], e[3 * sk]};
            }
        }
        S[m] = s;
    }
    // lazy decay, as in the narrow kernel: the registers hold S / 2^lg
    constexpr float LG_MIN = std::is_same<T, bf16_t>::value ? -60.f : 1.f;
    float lg = 0.f;

    const int tr_i = c16 >> 2, tr_j = c16 & 3;
    const int k_tr = (g * 64 + 4 * tr_i + ((tr_j + g) & 3)) * 8;
    int v_tr;
    {
        const int c = 2 * w + (tr_j >> 1);
        v_tr = (g * 64 + 16 * (c >> 2) + 4 * tr_i + ((c + g) & 3)) * 8 + 4 * (tr_j & 1);
    }

    auto step = [&](const char* kbuf, const char* vbuf, const char* rec, int istep) {
        const V8* sK = (const V8*)kbuf;
        const V8* sQ = (const V8*)(smem + W2_Q);
        const T* sV = (const T*)vbuf;
        const T* sKt = (const T*)kbuf;
        const char* sX = rec + W2_RX;
        const char* sP = smem + W2_P;
        const float* sTab = (const float*)(rec + W2_RTAB);
        auto fence = [] { __builtin_amdgcn_sched_barrier(0); };

        // fragment f = (t-tile f/8, key features 32s .. 32s+31 with s = f%8) of k or of q, each in a ring of four registers
        // sets: a region multiplies two fragments and fetches the two of the next region
        auto fidx = [&](int f) { return ((f & 7) >> 2) * 1024 + (f >> 3) * 256 + 16 * (f & 3) + a_off; };
        V8 ak[4], aq[4];
        auto Fk = [&](int f) { if (f < 32) ak[f & 3] = sK[fidx(f)]; };
        auto Fq = [&](int f) { if constexpr (FULL) { if (f < 32) aq[f & 3] = sQ[fidx(f)]; } };
        f32x4 ks[4], ao[4];
        V8 Sb[8];
        auto Mk = [&](int f) { ks[f >> 3] = Mma<T>::run(ak[f & 3], Sb[f & 7], (f & 7) ? ks[f >> 3] : f32x4{0.f, 0.f, 0.f, 0.f}); };
        auto Mq = [&](int f) { if constexpr (FULL) ao[f >> 3] = Mma<T>::run(Sb[f & 7], aq[f & 3], (f & 7) ? ao[f >> 3] : f32x4{0.f, 0.f, 0.f, 0.f}); };
        auto KK = [&](int r) { Fk(2 * r + 2); Fk(2 * r + 3); Mk(2 * r); Mk(2 * r + 1); };       // region r of the k products
        auto QQ = [&](int r) { Fq(2 * r + 2); Fq(2 * r + 3); Mq(2 * r); Mq(2 * r + 1); };       // region r of the q products
        V4 vv[4];
        V8 ax[4][2], ap[4][2];
        auto FV = [&](int tt) { vv[tt] = Mma<T>::tr_read(sV + tt * 2048 + v_tr); };
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
        // k^T operands of the state update, u = 16 sp2 + m (t-tile pair sp2, key tile m), in a ring of 8, fetched 6 ahead
        V8 kt[8];
        auto FK = [&](int u) {
            if (u >= 32) return;
            const int sp2 = u >> 4, m = u & 15;
            const T* a = sKt + (m >> 3) * 8192 + sp2 * 4096 + 128 * ((m & 7) >> 1) + 4 * (m & 1) + k_tr;
            kt[u & 7] = join<V8>(Mma<T>::tr_read(a), Mma<T>::tr_read(a + 2048));
        };
        float gamma, vscale;
        V8 Db[2], Vn[2], Vg[2];
        auto TD = [&](int tt) {
            const f32x4 eg = *(const f32x4*)(sTab + TAB_EG + 16 * tt + 4 * g) * gamma;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float x = (!FULL && v_zero) ? 0.f : to_f32(vv[tt][r]);      // (full runs always have their v)
                Db[tt >> 1][(tt & 1) * 4 + r] = from_f32<T>(x - eg[r] * ks[tt][r]);
            }
        };
        f32x4 vn[4], oacc[4];
        auto TXa = [&](int tt) {
            vn[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int sp2 = 0; sp2 <= (tt >> 1); ++sp2) vn[tt] = Mma<T>::run(ax[tt][sp2], Db[sp2], vn[tt]);
        };
        auto TXb = [&](int tt) {
            const f32x4 dec = *(const f32x4*)(sTab + TAB_DEC + 16 * tt + 4 * g) * vscale;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                Vn[tt >> 1][(tt & 1) * 4 + r] = from_f32<T>(vn[tt][r]);
                Vg[tt >> 1][(tt & 1) * 4 + r] = from_f32<T>(vn[tt][r] * dec[r]);
            }
        };
        auto TPa = [&](int tt) {
            if constexpr (FULL) {
                const float gam = sTab[TAB_SG + 16 * tt + c16] * gamma;
                oacc[tt] = ao[tt] * gam;
#pragma unroll
                for (int sp2 = 0; sp2 <= (tt >> 1); ++sp2) oacc[tt] = Mma<T>::run(Vn[sp2], ap[tt][sp2], oacc[tt]);
            }
        };
        auto TPb = [&](int tt) {
            if constexpr (FULL) {
                V4 o4;
#pragma unroll
                for (int r = 0; r < 4; ++r) o4[r] = from_f32<T>(oacc[tt][r]);
                *(V4*)(otile + (16 * tt + c16) * W2_OT_PITCH + (16 * w + 4 * g) * 2) = o4;
            }
        };
        auto UU = [&](int j) {                   // two products of the state update, and the operands of two later ones
            FK(2 * j + 6); FK(2 * j + 7);
            S[(2 * j) & 15] = Mma<T>::run(kt[(2 * j) & 7], Vg[j >> 3], S[(2 * j) & 15]);
            S[(2 * j + 1) & 15] = Mma<T>::run(kt[(2 * j + 1) & 7], Vg[j >> 3], S[(2 * j + 1) & 15]);
        };

        Fk(0); Fk(1);
#pragma unroll
        for (int s = 0; s < 8; ++s)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                Sb[s][r] = from_f32<T>(S[2 * s][r]);
                Sb[s][4 + r] = from_f32<T>(S[2 * s + 1][r]);
            }
        gamma = fast_exp2(lg);
        const float lg_try = lg + sTab[TAB_GLAST];
        const bool lazy = lg_try >= LG_MIN;
        vscale = lazy ? fast_exp2(-lg_try) : 1.f;
        // the decay fold (rare; a scalar branch): the products below read the bf16 copy made above, the update the folded state
        if (__builtin_amdgcn_readfirstlane((int)lazy) == 0) {
            const float fold = fast_exp2(lg_try);
#pragma unroll
            for (int m = 0; m < 16; ++m) S[m] *= fold;
        }
        lg = lazy ? lg_try : 0.f;
        fence();
        // ---- The products with k come first: they head the chain that the next step waits for (k S -> D -> v_new -> state
        // update), and q of this chunk may still be on its way.  The update from t-tiles 0, 1 starts while tiles 2, 3 are
        // still being multiplied; the products with q, P and the output fill the second half of the step. ----
        KK(0); FV(0); fence();
        KK(1); FV(1); fence();
        KK(2); FX(0); fence();
        KK(3); FX(1); fence();
        KK(4); TD(0); FK(0); FK(1); fence();
        KK(5); FV(2); FK(2); FK(3); fence();
        KK(6); FV(3); FK(4); FK(5); fence();
        KK(7); fence();
        KK(8); TD(1); fence();
        KK(9); TXa(0); TXa(1); fence();
        KK(10); TXb(0); TXb(1); fence();
        KK(11); UU(0); fence();
        if constexpr (FULL) { while (*qcount < istep + 1) __builtin_amdgcn_s_sleep(1); }      // q of this chunk (normally long there)
        asm volatile("" ::: "memory");                                // (no read of the tile may move in front of the poll)
        Fq(0); Fq(1);
        KK(12); UU(1); TD(2); FX(2); fence();
        KK(13); UU(2); QQ(0); fence();
        KK(14); UU(3); QQ(1); FX(3); fence();
        KK(15); UU(4); QQ(2); fence();
        TD(3); UU(5); QQ(3); fence();
        TXa(2); TXa(3); UU(6); QQ(4); fence();
        TXb(2); TXb(3); UU(7); QQ(5); fence();
        if constexpr (FULL) { while (*pcount < 4 * (istep + 1)) __builtin_amdgcn_s_sleep(1); }      // P of this chunk
        asm volatile("" ::: "memory");
        FP(0); FP(1);
        UU(8); QQ(6); fence();
        UU(9); QQ(7); TPa(0); fence();
        UU(10); QQ(8); TPa(1); TPb(0); FP(2); fence();
        UU(11); QQ(9); TPb(1); FP(3); fence();
        UU(12); QQ(10); fence();
        QQ(11); TPa(2); fence();
        QQ(12); TPb(2); fence();
        QQ(13); fence();
        QQ(14); fence();
        QQ(15); fence();
        TPa(3); fence();
        TPb(3); fence();
        lds_barrier();                                          // B1: q, v, the record and P are free, the output tile is complete
        UU(13); UU(14); UU(15); fence();
        lds_barrier();                                          // B2: k of this stage is free, k, v and the record of the next chunk are complete
    };
    if (nsteps > 0) {
        lds_barrier();                                          // B0
        for (int64_t i = 0; i < nsteps; ++i)
            step(smem + W2_KB + (int)(i & 1) * 32768, smem + W2_V + (int)(i & 1) * 16384, smem + W2_REC + (int)(i & 1) * W2_REC_BYTES,
                 (int)i);
    }

    if (dst) {
        const float gamma = fast_exp2(lg);
        const int sk = dst_user ? (vfirst ? 1 : V) : buf_pitch, sv = dst_user ? (vfirst ? K : 1) : 1;
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            const int kk = 32 * (m >> 1) + 8 * g + 4 * (m & 1);
            const f32x4 s = S[m] * gamma;
            if (kk < (dst_user ? K : W2_KD) && vc < (dst_user ? V : buf_pitch)) {
                float* e = dst + (int64_t)kk * sk + (int64_t)vc * sv;
#pragma unroll
                for (int r = 0; r < 4; ++r) e[r * sk] = s[r];
            }
        }
    }
}

// S_in[j+1] = M_j S_in[j] + S_loc,j for j = 1 .. nseg-2, with S_in[1] = S_loc,0 (the run of segment 0 started from the true
// initial state), for the 256-row states of wide keys.  fp32 throughout (fp32 matrix cores): one workgroup per (sequence,
// head, slab of 16 value columns) keeps the slab transposed in LDS and stages M_j by halves of 128 rows; wave w takes
// the key tiles 2w, 2w+1 of a half.  Buffers per (sequence, head, segment): S_loc [256][VP], M [256][256], S_in [256][VP].
constexpr int M2P = W2_KD + 4;                     // pitch of the staged rows (floats): conflict-free 16-byte reads
constexpr size_t MERGE256_SMEM = (128 * M2P + 16 * M2P) * 4;

__global__ __launch_bounds__(256) void gdn_segment_merge256_kernel(SegmentPlan sp, float* seg, int64_t NH, int HV, int64_t NT, int VP,
                                                                   size_t seg_floats) {
    extern __shared__ __align__(16) char smem[];
    float* sM = (float*)smem;                      // [128 rows of a half][M2P]
    float* sSt = sM + 128 * M2P;                   // [16 columns][M2P]: the current S_in slab, transposed
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    const int slabs = VP / 16;
    const int64_t inh = blockIdx.x / slabs;
    const int v0 = (int)(blockIdx.x % slabs) * 16;
    if (inh >= NH) return;
    if (sp.bound && !needs_exact_segments(sp, sp.bound + (inh / HV) * NT * HV + inh % HV, HV, lane)) return;      // all segments start warm
    const int nseg = sp.nseg;
    auto sloc = [&](int j) { return seg + (size_t)(inh * nseg + j) * seg_floats; };
    auto mseg = [&](int j) { return sloc(j) + (size_t)W2_KD * VP; };
    auto sin = [&](int j) { return mseg(j) + (size_t)W2_KD * W2_KD; };
    // this wave's part of a slab: per half the key tiles 2w, 2w+1 in C/D layout (column c16, rows 4g .. 4g+3)
    auto row_of = [&](int half, int i) { return 128 * half + 16 * (2 * w + i) + 4 * g; };
    f32x4 x[2][2];
    auto publish = [&](int j) {                    // x becomes S_in[j]: to the other waves (transposed) and to memory
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                *(f32x4*)(sSt + c16 * M2P + row_of(half, i)) = x[half][i];
#pragma unroll
                for (int r = 0; r < 4; ++r) sin(j)[(size_t)(row_of(half, i) + r) * VP + v0 + c16] = x[half][i][r];
            }
    };
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) x[half][i][r] = sloc(0)[(size_t)(row_of(half, i) + r) * VP + v0 + c16];
    publish(1);
    for (int j = 1; j + 1 < nseg; ++j) {
        f32x4 y[2][2];
        for (int half = 0; half < 2; ++half) {
            __syncthreads();                        // the slab is complete; the last reads of the previous half are done
            const float* M = mseg(j) + (size_t)128 * half * W2_KD;
            for (int i0 = 0; i0 < 32; i0 += 8) {
                f32x4 pre[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int idx = tid + 256 * (i0 + i);                   // 64 pieces of 16 bytes per row
                    pre[i] = *(const f32x4*)(M + (size_t)(idx >> 6) * W2_KD + (idx & 63) * 4);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int idx = tid + 256 * (i0 + i);
                    *(f32x4*)(sM + (idx >> 6) * M2P + (idx & 63) * 4) = pre[i];
                }
            }
            __syncthreads();                        // this half of M_j is in LDS
            f32x4 acc[2][2];                        // two accumulation chains per tile (even / odd blocks)
#pragma unroll
            for (int i = 0; i < 2; ++i) acc[i][0] = acc[i][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const f32x4 b = *(const f32x4*)(sSt + c16 * M2P + 16 * q + 4 * g);
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const f32x4 a = *(const f32x4*)(sM + (16 * (2 * w + i) + c16) * M2P + 16 * q + 4 * g);
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][q & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], acc[i][q & 1], 0, 0, 0);
                }
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                f32x4 sl;
#pragma unroll
                for (int r = 0; r < 4; ++r) sl[r] = sloc(j)[(size_t)(row_of(half, i) + r) * VP + v0 + c16];
                y[half][i] = acc[i][0] + acc[i][1] + sl;
            }
        }
        __syncthreads();                            // all waves have read the slab S_in[j]
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int i = 0; i < 2; ++i) x[half][i] = y[half][i];
        publish(j + 1);
    }
}

template <typename T, bool FULL>
static int launch_wide256_kind(const ChunkParams& p, int NVB, const SegmentPlan& sp, int64_t blocks, hipStream_t stream) {
    auto kern = gdn_chunk_wide256_kernel<T, FULL>;
    static SmemAttrDone attr_done;       // per instantiation
    if (int rc = ensure_dynamic_smem((const void*)kern, W2_SMEM, attr_done, "hipFuncSetAttribute(wide256)")) return rc;
    if (blocks >= (1ll << 31)) { set_error("gdn_chunk_fwd: too many workgroups for one launch"); return GDN_ERR_UNSUPPORTED; }
    if (blocks <= 0) return GDN_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(W2_THREADS), W2_SMEM, stream, p, NVB, sp);
    return check_launch("gdn_chunk_wide256_kernel");
}

template <typename T>
int launch_wide256(const ChunkParams& p, hipStream_t stream) {
    const int NVB = (p.V + W2_VB - 1) / W2_VB;
    const int64_t G = p.HV / p.H;
    SegmentPlan sp = {};
    sp.nseg = plan_segments256(p.N, p.H, p.HV, p.V, p.NT, p.cu_seqlens == nullptr, p.flags);
    sp.seg_chunks = 1 << 30;
    if (sp.nseg > 1) {
        sp.seg_chunks = (int)((p.NT + sp.nseg - 1) / sp.nseg);
        // Segments start warm where the decay allows it; the first pass and the merge then only serve the heads that need
        // exact start states, and their workgroups for the other heads return at once.
        if (!(p.flags & GDN_FLAG_SCAN_NO_WARM)) {
            sp.bound = p.ws.Bound;
            sp.warm_cap = std::min(WARM_CAP_MAX, sp.seg_chunks + sp.seg_chunks / 4 + 6);
        }
        // pass 1: per (sequence, q/k head, segment but the last) the S runs of its value heads' column blocks, then the M runs
        if (int rc = launch_wide256_kind<T, false>(p, NVB, sp, (p.N * p.H * (sp.nseg - 1) + 7) / 8 * 8 * G * (NVB + W2_KD / W2_VB), stream)) return rc;
        static SmemAttrDone attr_done;
        if (int rc = ensure_dynamic_smem((const void*)gdn_segment_merge256_kernel, MERGE256_SMEM, attr_done, "hipFuncSetAttribute(merge256)")) return rc;
        const int VP = NVB * W2_VB;
        hipLaunchKernelGGL(gdn_segment_merge256_kernel, dim3((unsigned)(p.NH * (VP / 16))), dim3(256), MERGE256_SMEM, stream, sp, p.ws.Seg,
                           p.NH, p.HV, p.NT, VP, seg256_floats(p.V));
        if (int rc = check_launch("gdn_segment_merge256_kernel")) return rc;
    }
    return launch_wide256_kind<T, true>(p, NVB, sp, (p.N * p.H * sp.nseg + 7) / 8 * 8 * G * NVB, stream);
}

template int launch_wide256<bf16_t>(const ChunkParams&, hipStream_t);
template int launch_wide256<f16_t>(const ChunkParams&, hipStream_t);

}  // namespace gdn
