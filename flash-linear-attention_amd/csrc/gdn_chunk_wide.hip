// Sequential stage of the chunked prefill, "wide" form: one workgroup per (sequence, v-head,
// segment of consecutive chunks) holds the WHOLE fp32 state S[128, 128] in registers.
//
// Ten waves.  Eight compute waves: wave w owns value columns 16w .. 16w+15 for all key rows.
// Nothing of the recurrence crosses waves: bf16(S) and bf16(v_new) are the B operands of this
// wave's own next products (same lanes, C/D layout == operand layout), so the dependent chain
// S -> w S -> v_new -> k^T v_new -> S runs in registers.  Two waves per SIMD let one wave's
// vector-ALU work overlap the other's matrix instructions.  The compute waves issue no global
// memory instruction inside the loop.
// Two copy waves move everything else: what the compute waves share are the A operands (w, q,
// k^T, P, u fragments and the gate tables, 71 KB per chunk); they are copied verbatim from the
// workspace into a double-buffered LDS stage by asynchronous global->LDS loads that use no
// registers, and the output tile of a chunk goes LDS -> registers -> global in 256-byte rows.
// Two barriers per chunk (after each half of a step) are the only synchronisation.
//
// The same kernel serves the segment-parallel evaluation of long sequences
// (S_out = M S_in + S_loc per segment):
//   pass 1  state only (no q / P / output), started from the true initial state (first
//           segment), from zero (S_loc) or from the identity with u = 0 (the transition M);
//   merge   S_in[j+1] = M_j S_in[j] + S_loc,j in fp32 (gdn_segment_merge_kernel);
//   pass 2  full evaluation of every segment from its merged initial state.
#include "gdn_chunk_common.h"

namespace gdn {

// LDS stage = verbatim copy of one chunk's workspace fragments
constexpr int STG_W = 0, STG_Q = 16384, STG_KT = 32768, STG_P = 49152, STG_U = 55296, STG_TAB = 71680;
constexpr int STG_BYTES = 72704;                  // W 16K, Q 16K, k^T 16K, P 6K (the 6 non-zero pieces), u 16K, tables 1K
constexpr int OT_PITCH = 272;                     // bytes per token row of the output tile (256 B + pad: conflict-free 8-byte writes)
constexpr int OT_BYTES = 64 * OT_PITCH;           // 17 408 B
constexpr size_t WIDE_SMEM = 2 * STG_BYTES + OT_BYTES;       // 162 816 B of the CU's 163 840: one workgroup per CU
constexpr int CW = 8;                             // compute waves
constexpr int WIDE_THREADS = (CW + 2) * 64;
// P pieces (t-tile tt, column pair sp2) -> slot in the stage; (0,1) and (1,1) are identically zero and not staged
__host__ __device__ constexpr int p_slot(int tt, int sp2) { return tt < 2 ? tt : 2 + 2 * (tt - 2) + sp2; }

// kind of run
constexpr int WIDE_WHOLE = 0;     // whole sequences, user h0 -> o, ht
constexpr int WIDE_PASS1 = 1;     // per segment: S_loc / M into the segment buffers
constexpr int WIDE_PASS2 = 2;     // per segment: from merged S_in -> o (last segment also ht)

// Asynchronous copy of 1 KB (16 bytes per lane) from global memory straight into LDS at the
// wave-uniform byte offset `lds_off` (+ 16 * lane).  Issued from inline assembly on purpose:
// the compiler then keeps no account of it, and completion is awaited explicitly with
// s_waitcnt vmcnt before the barrier that publishes the data.
// `gsrc` is the wave-uniform source of the 1 KB piece (scalar base), `lane_off` = 16 * lane.
__device__ __forceinline__ void copy_1k_to_lds(const char* gsrc, uint32_t lane_off, uint32_t lds_off) {
    lds_off = __builtin_amdgcn_readfirstlane(lds_off);          // wave-uniform by construction; make them scalars
    const uint64_t g = (uint64_t)gsrc;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)g), hi = __builtin_amdgcn_readfirstlane((uint32_t)(g >> 32));
    const uint64_t gs = ((uint64_t)hi << 32) | lo;
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_off), "v"(lane_off), "s"(gs));
}

template <int N>
__device__ __forceinline__ void wait_vm_at_most() {
    static_assert(N >= 0 && N <= 63, "the vector-memory counter has 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

template <typename T, bool FULL>
__global__ __launch_bounds__(WIDE_THREADS) void gdn_chunk_wide_kernel(ChunkParams p, SegmentPlan sp) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];

    const int tid = threadIdx.x, lane = tid & 63, c16 = lane & 15, g = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);       // scalar: the roles below branch on it
    const int H = p.H, HV = p.HV;
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    const bool vfirst = p.flags & GDN_FLAG_STATE_V_FIRST;

    // ---- which (sequence, head, segment) and what to start from / write to ----
    int64_t inh;
    int seg;
    int init = 0;                 // 0: from `src` (NULL = zero state), 1: identity, 2: zero
    bool u_zero = false, src_user = false, dst_user = false;
    const float* src = nullptr;
    float* dst = nullptr;
    if (sp.kind == WIDE_WHOLE) {
        inh = blockIdx.x; seg = 0;
        src = p.h0 ? p.h0 + inh * 16384 : nullptr; src_user = true;
        dst = p.ht ? p.ht + inh * 16384 : nullptr; dst_user = true;
    } else if (sp.kind == WIDE_PASS1) {
        const int per = 2 * sp.nseg - 3;                    // S runs of segments 0..nseg-2, M runs of 1..nseg-2
        inh = blockIdx.x / per;
        const int idx = (int)(blockIdx.x % per);
        if (idx < sp.nseg - 1) {
            seg = idx;
            if (seg == 0) { src = p.h0 ? p.h0 + inh * 16384 : nullptr; src_user = true; }
            else init = 2;
            dst = sp.sloc + (inh * sp.nseg + seg) * 16384;
        } else {
            seg = idx - (sp.nseg - 1) + 1;
            init = 1; u_zero = true;
            dst = sp.mseg + (inh * sp.nseg + seg) * 16384;
        }
    } else {
        inh = blockIdx.x / sp.nseg;
        seg = (int)(blockIdx.x % sp.nseg);
        if (seg == 0) { src = p.h0 ? p.h0 + inh * 16384 : nullptr; src_user = true; }
        else src = sp.sin + (inh * sp.nseg + seg) * 16384;
        if (seg == sp.nseg - 1 && p.ht) { dst = p.ht + inh * 16384; dst_user = true; }
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
    const int64_t it0 = (int64_t)seg * sp.seg_chunks;
    const int64_t it1 = min(nt, it0 + sp.seg_chunks);
    const int64_t nsteps = it1 - it0;                       // may be <= 0 for an empty sequence
    const int64_t lastc = it1 - 1;
    char* otile = smem + 2 * STG_BYTES;                     // [64 token rows][OT_PITCH]

    // =====================================================================================
    // Copy waves.  Step i (chunk it = it0 + i, stage cur = i & 1) has two phases, separated by
    // the workgroup barriers B1 (after the first half) and B2 (after the second half):
    //   phase A  compute waves read w, q, P, u, tables of stage cur and write the output tile
    //   phase B  compute waves read k^T of stage cur
    // Loads complete in issue order, so "at most N operations outstanding" proves that all but
    // the N newest have landed; outstanding stores only make such a wait longer.
    // =====================================================================================
    if (w >= CW) {
        if (nsteps <= 0) return;
        const char* Wf = (const char*)p.ws.Wf;
        const char* Uf = (const char*)p.ws.Uf;
        const char* KTf = (const char*)p.ws.KTf;
        const char* Pf = (const char*)p.ws.Pf;
        const char* Qf = (const char*)p.ws.Qf;
        const char* Tab = (const char*)p.ws.Tab;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
        const uint32_t l16 = lane * 16;
        if (w == CW) {
            // ---- first-half operands: NOPS one-KB pieces per chunk, pieces [0, XA) are issued in
            // phase B of step c-2 and the rest in phase A of step c-1 (their LDS region is free from
            // B1 of step c-2 on); all must have landed at B2 of step c-1.
            constexpr int NOPS = FULL ? 55 : 33;
            constexpr int XA = 16;
            auto piece = [&](auto op_c, int64_t it, int stage) {
                constexpr int op = decltype(op_c)::value;
                const int64_t ci = boh + it;
                const int64_t chv = ci * HV + hv, ch = ci * H + h;
                const uint32_t base = lds0 + stage * STG_BYTES;
                if constexpr (op < 16) copy_1k_to_lds(Wf + chv * (WS_W * 2) + op * 1024, l16, base + STG_W + op * 1024);
                else if constexpr (op < 32) copy_1k_to_lds(Uf + chv * (WS_U * 2) + (op - 16) * 1024, l16, base + STG_U + (op - 16) * 1024);
                else if constexpr (op == 32) copy_1k_to_lds(Tab + chv * (WS_TAB * 4), l16, base + STG_TAB);
                else if constexpr (op < 49) copy_1k_to_lds(Qf + ch * (WS_Q * 2) + (op - 33) * 1024, l16, base + STG_Q + (op - 33) * 1024);
                else {
                    // P: workspace pieces 0,2,4,5,6,7 (the others are zero) go to slots 0..5
                    constexpr int slot = op - 49, srcp = slot < 2 ? 2 * slot : slot + 2;
                    copy_1k_to_lds(Pf + chv * (WS_P * 2) + srcp * 1024, l16, base + STG_P + slot * 1024);
                }
            };
            auto issue = [&](auto from_c, auto to_c, int64_t it, int stage) {
                constexpr int from = decltype(from_c)::value, to = decltype(to_c)::value;
                [&]<int... I>(std::integer_sequence<int, I...>) {
                    (piece(std::integral_constant<int, from + I>{}, it, stage), ...);
                }(std::make_integer_sequence<int, to - from>{});
            };
            std::integral_constant<int, 0> c0;
            std::integral_constant<int, XA> cx;
            std::integral_constant<int, NOPS> cn;
            issue(c0, cn, it0, 0);
            issue(c0, cx, min(it0 + 1, lastc), 1);
            wait_vm_at_most<XA>();
            lds_barrier();                                                  // B0: stage 0 is complete
            for (int64_t i = 0; i < nsteps; ++i) {
                const int64_t it = it0 + i;
                const int cur = (int)(i & 1);
                issue(cx, cn, min(it + 1, lastc), cur ^ 1);
                lds_barrier();                                              // B1
                issue(c0, cx, min(it + 2, lastc), cur);
                wait_vm_at_most<XA>();                                      // the first-half operands of chunk it+1 have landed
                lds_barrier();                                              // B2
            }
            wait_vm_at_most<0>();                                           // no copy may land in LDS after this workgroup has gone
        } else {
            // ---- k^T (16 pieces per chunk, issued in phase A one step ahead) and the output rows
            T* og = (T*)p.o;
            u32x4 orow[16];                                                 // output tile of the previous chunk
            auto issue_kt = [&](int64_t it, int stage) {
                const int64_t ch = (boh + it) * H + h;
                const uint32_t base = lds0 + stage * STG_BYTES;
#pragma unroll
                for (int j = 0; j < 16; ++j) copy_1k_to_lds(KTf + ch * (WS_KT * 2) + j * 1024, l16, base + STG_KT + j * 1024);
            };
            // one instruction stores 4 token rows of 256 bytes
            auto store_rows = [&](int64_t it) {
                const int valid = (int)min((int64_t)CH, len - it * CH);
                int64_t stride = (int64_t)HV * 128 * 4;                     // elements between rows 4 apart
                asm volatile("" : "+s"(stride));                            // keep the 16 row addresses out of long-lived registers
                T* dstp = og + ((bos + it * CH + g) * HV + hv) * 128 + c16 * 8;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    if (4 * j + g < valid) *(u32x4*)dstp = orow[j];
                    dstp += stride;
                }
            };
            issue_kt(it0, 0);
            wait_vm_at_most<0>();
            lds_barrier();                                                  // B0
            for (int64_t i = 0; i < nsteps; ++i) {
                const int64_t it = it0 + i;
                const int cur = (int)(i & 1);
                issue_kt(min(it + 1, lastc), cur ^ 1);                      // that region was last read before B2 of the previous step
                if constexpr (FULL) {
                    if (i > 0) store_rows(it - 1);
                    // k^T of this chunk was issued one step ago; newer than it are the stores of chunks
                    // it-2 and it-1 (16 each, all rows of those chunks are valid) and the k^T just issued
                    if (i >= 2) wait_vm_at_most<48>();
                    else if (i == 1) wait_vm_at_most<32>();
                } else {
                    wait_vm_at_most<16>();
                }
                lds_barrier();                                              // B1
                if constexpr (FULL) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) orow[j] = *(const u32x4*)(otile + (4 * j + g) * OT_PITCH + c16 * 16);
                }
                lds_barrier();                                              // B2 (waits for the tile reads)
            }
            if constexpr (FULL) store_rows(lastc);
            wait_vm_at_most<0>();
        }
        return;
    }

    // =====================================================================================
    // Compute waves
    // =====================================================================================
    // ---- state: all key rows, value columns 16w .. 16w+15, C/D layout ----
    f32x4 S[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        const int kk = 16 * m + 4 * g, vc = 16 * w + c16;
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        if (init == 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] = (kk + r == vc) ? 1.f : 0.f;
        } else if (init == 0 && src) {
            if (src_user && vfirst) s = *(const f32x4*)(src + vc * 128 + kk);
            else s = f32x4{src[kk * 128 + vc], src[(kk + 1) * 128 + vc], src[(kk + 2) * 128 + vc], src[(kk + 3) * 128 + vc]};
        }
        S[m] = s;
    }

    // Lazy decay: registers hold S / Gamma, Gamma = 2^lg one scalar per workgroup (see the slab kernel).
    constexpr float LG_MIN = std::is_same<T, bf16_t>::value ? -60.f : 1.f;
    float lg = 0.f;

    V8 Vg[2];              // v_new decayed to the chunk end, B operand of the state update (first half -> second half)
    auto first_half = [&](const char* st) {
        const V8* sW = (const V8*)(st + STG_W);
        const V8* sQ = (const V8*)(st + STG_Q);
        const V8* sP = (const V8*)(st + STG_P);
        const V4* sU = (const V4*)(st + STG_U);
        const float* sTab = (const float*)(st + STG_TAB);
        // (a) the state as B operand: pairs of key tiles (2s, 2s+1)
        V8 Sb[4];
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                Sb[s][r] = from_f32<T>(S[2 * s][r]);
                Sb[s][4 + r] = from_f32<T>(S[2 * s + 1][r]);
            }
        const float gamma = fast_exp2(lg);
        const float lg_try = lg + sTab[128];
        const bool lazy = lg_try >= LG_MIN;
        const float vscale = lazy ? fast_exp2(-lg_try) : 1.f;
        V8 Vn[2];
        // two t-tiles at a time: w S -> v_new, and the output rows of those tiles
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            f32x4 av[2], ao[2];
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const int tt = 2 * hf + t2;
                av[t2] = f32x4{0.f, 0.f, 0.f, 0.f};
                ao[t2] = f32x4{0.f, 0.f, 0.f, 0.f};
                V8 aw[4], aq[4];
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    aw[s] = sW[(tt * 4 + s) * 64 + lane];
                    if constexpr (FULL) aq[s] = sQ[(tt * 4 + s) * 64 + lane];
                }
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    av[t2] = Mma<T>::run(aw[s], Sb[s], av[t2]);
                    if constexpr (FULL) ao[t2] = Mma<T>::run(Sb[s], aq[s], ao[t2]);     // transposed tile
                }
            }
            // v_new = u - w S, plain (for the output) and decayed to the chunk end (for the state)
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const int tt = 2 * hf + t2;
                const f32x4 dec = *(const f32x4*)(sTab + 16 * tt + 4 * g) * vscale;
                const V4 u4 = sU[(w * 4 + tt) * 64 + lane];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float uu = u_zero ? 0.f : to_f32(u4[r]);
                    const float vn = uu - gamma * av[t2][r];
                    Vn[hf][t2 * 4 + r] = from_f32<T>(vn);
                    Vg[hf][t2 * 4 + r] = from_f32<T>(vn * dec[r]);
                }
            }
            // o^T = scale 2^G (q S)^T + (P v_new)^T; each lane holds 4 consecutive value columns of a token row
            if constexpr (FULL) {
#pragma unroll
                for (int t2 = 0; t2 < 2; ++t2) {
                    const int tt = 2 * hf + t2;
                    const float gam = sTab[64 + 16 * tt + c16] * gamma;
                    f32x4 acc = ao[t2] * gam;
#pragma unroll
                    for (int sp2 = 0; sp2 <= hf; ++sp2) acc = Mma<T>::run(Vn[sp2], sP[p_slot(tt, sp2) * 64 + lane], acc);
                    V4 o4;
#pragma unroll
                    for (int r = 0; r < 4; ++r) o4[r] = from_f32<T>(acc[r]);
                    *(V4*)(otile + (16 * tt + c16) * OT_PITCH + (16 * w + 4 * g) * 2) = o4;
                }
            }
        }
        if (__builtin_amdgcn_readfirstlane((int)lazy) == 0) {       // scalar branch: rare, must not be if-converted
            const float fold = fast_exp2(lg_try);
#pragma unroll
            for (int m = 0; m < 8; ++m) S[m] *= fold;
        }
        lg = lazy ? lg_try : 0.f;
    };
    // S += k^T (v_new decayed)
    auto second_half = [&](const char* st) {
        const V8* sKT = (const V8*)(st + STG_KT);
#pragma unroll
        for (int m = 0; m < 8; ++m)
#pragma unroll
            for (int sp2 = 0; sp2 < 2; ++sp2) S[m] = Mma<T>::run(sKT[(m * 2 + sp2) * 64 + lane], Vg[sp2], S[m]);
    };
    if (nsteps > 0) {
        lds_barrier();                                          // B0: the copy waves have filled stage 0
        for (int64_t i = 0; i < nsteps; ++i) {
            const char* st = smem + (i & 1) * STG_BYTES;
            first_half(st);
            lds_barrier();                                      // B1
            second_half(st);
            lds_barrier();                                      // B2
        }
    }

    if (dst) {
        const float gamma = fast_exp2(lg);
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const int kk = 16 * m + 4 * g, vc = 16 * w + c16;
            const f32x4 s = S[m] * gamma;
            if (dst_user && vfirst) *(f32x4*)(dst + vc * 128 + kk) = s;
            else {
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[(kk + r) * 128 + vc] = s[r];
            }
        }
    }
}

// S_in[j+1] = M_j S_in[j] + S_loc,j for j = 1 .. nseg-2, with S_in[1] = S_loc,0 (the run of segment 0
// started from the true initial state).  fp32 throughout (fp32 matrix cores): one workgroup
// per (sequence, head, slab of 16 value columns); M_j is staged in LDS.
constexpr int MP = 132;                            // pitch of the staged M rows (floats)
constexpr size_t MERGE_SMEM = (128 * MP + 128 * 16) * 4;

__global__ __launch_bounds__(256) void gdn_segment_merge_kernel(SegmentPlan sp) {
    extern __shared__ __align__(16) char smem[];
    float* sM = (float*)smem;                      // [128][MP]
    float* sS = sM + 128 * MP;                     // [128][16] current S_in slab
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    const int64_t inh = blockIdx.x >> 3;
    const int v0 = (int)(blockIdx.x & 7) * 16;
    const int nseg = sp.nseg;
    // S_in[1] = S_loc,0
    for (int idx = tid; idx < 128 * 16; idx += 256) {
        const int kk = idx >> 4, c = idx & 15;
        const float x = sp.sloc[(inh * nseg + 0) * 16384 + kk * 128 + v0 + c];
        sS[idx] = x;
        sp.sin[(inh * nseg + 1) * 16384 + kk * 128 + v0 + c] = x;
    }
    for (int j = 1; j + 1 < nseg; ++j) {
        const float* M = sp.mseg + (inh * nseg + j) * 16384;
        __syncthreads();                            // previous readers of sM are done; sS is complete
        for (int idx = tid; idx < 128 * 32; idx += 256) {
            const int row = idx >> 5, c4 = (idx & 31) * 4;
            *(f32x4*)(sM + row * MP + c4) = *(const f32x4*)(M + row * 128 + c4);
        }
        __syncthreads();
        f32x4 acc[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) acc[i] = mm16_f32(sM + (16 * (2 * w + i)) * MP, MP, sS, 16, 32, c16, g);
        __syncthreads();                            // all waves have read sS
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int kk = 16 * (2 * w + i) + 4 * g + r;
                const float x = acc[i][r] + sp.sloc[(inh * nseg + j) * 16384 + kk * 128 + v0 + c16];
                sS[kk * 16 + c16] = x;
                sp.sin[(inh * nseg + j + 1) * 16384 + kk * 128 + v0 + c16] = x;
            }
    }
}

template <typename T, bool FULL>
static int launch_wide_kind(const ChunkParams& p, const SegmentPlan& sp, int64_t blocks, hipStream_t stream) {
    auto kern = gdn_chunk_wide_kernel<T, FULL>;
    static bool attr_done = false;
    if (!attr_done) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)WIDE_SMEM) != hipSuccess)
            return check_launch("hipFuncSetAttribute(wide)");
        attr_done = true;
    }
    if (blocks <= 0) return GDN_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(WIDE_THREADS), WIDE_SMEM, stream, p, sp);
    return check_launch("gdn_chunk_wide_kernel");
}

template <typename T>
int launch_scan_wide(const ChunkParams& p, hipStream_t stream) {
    SegmentPlan sp = {};
    sp.kind = WIDE_WHOLE;
    sp.nseg = 1;
    sp.seg_chunks = 1 << 30;
    return launch_wide_kind<T, true>(p, sp, p.NH, stream);
}

template <typename T>
int launch_scan_segments(const ChunkParams& p, SegmentPlan sp, hipStream_t stream) {
    int rc;
    sp.kind = WIDE_PASS1;
    if ((rc = launch_wide_kind<T, false>(p, sp, p.NH * (2 * sp.nseg - 3), stream))) return rc;
    if (sp.nseg > 1) {
        static bool attr_done = false;
        if (!attr_done) {
            if (hipFuncSetAttribute((const void*)gdn_segment_merge_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)MERGE_SMEM) != hipSuccess)
                return check_launch("hipFuncSetAttribute(merge)");
            attr_done = true;
        }
        hipLaunchKernelGGL(gdn_segment_merge_kernel, dim3((unsigned)(p.NH * 8)), dim3(256), MERGE_SMEM, stream, sp);
        if ((rc = check_launch("gdn_segment_merge_kernel"))) return rc;
    }
    sp.kind = WIDE_PASS2;
    return launch_wide_kind<T, true>(p, sp, p.NH * sp.nseg, stream);
}

template int launch_scan_wide<bf16_t>(const ChunkParams&, hipStream_t);
template int launch_scan_wide<f16_t>(const ChunkParams&, hipStream_t);
template int launch_scan_segments<bf16_t>(const ChunkParams&, SegmentPlan, hipStream_t);
template int launch_scan_segments<f16_t>(const ChunkParams&, SegmentPlan, hipStream_t);

}  // namespace gdn
