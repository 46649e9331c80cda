// Sequential stage of the chunked prefill, "wide" form: one workgroup per (sequence, v-head,
// segment of consecutive chunks) holds the WHOLE fp32 state S[128, 128] in registers, wave w
// owning value columns 32w .. 32w+31 for all key rows.  Nothing of the recurrence crosses
// waves: bf16(S) and bf16(v_new) are the B operands of this wave's own next products (same
// lanes, C/D layout == operand layout), so the dependent chain S -> w S -> v_new -> k^T v_new
// -> S runs in registers with no barrier.  What the waves share are the A operands (w, q,
// k^T, P, u fragments and the gate tables, 73 KB per chunk): they are copied verbatim from the
// workspace into a double-buffered LDS stage by asynchronous global->LDS loads that use no
// registers and are issued one and a half steps before their data is needed; two barriers per
// chunk publish the two halves of a stage.
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
constexpr int OT_PITCH = 72;                      // bytes per row of a wave's private output tile (64 B + pad)
constexpr int OT_BYTES = 64 * OT_PITCH;           // 4608 B per wave
constexpr size_t WIDE_SMEM = 2 * STG_BYTES + 4 * OT_BYTES;   // 163 840 B = all of the CU's LDS: one workgroup per CU
// P pieces (t-tile tt, column pair sp2) -> slot in the stage; (0,1) and (1,1) are identically zero and not staged
__host__ __device__ constexpr int p_slot(int tt, int sp2) { return tt < 2 ? tt : 2 + 2 * (tt - 2) + sp2; }

// kind of run
constexpr int WIDE_WHOLE = 0;     // whole sequences, user h0 -> o, ht
constexpr int WIDE_PASS1 = 1;     // per segment: S_loc / M into the segment buffers
constexpr int WIDE_PASS2 = 2;     // per segment: from merged S_in -> o (last segment also ht)

// Asynchronous copy of 1 KB (16 bytes per lane) from global memory straight into LDS at the
// wave-uniform byte offset `lds_off` (+ 16 * lane).  Issued from inline assembly on purpose:
// the compiler then does not order later LDS reads of the OTHER stage behind it; completion
// is awaited explicitly (s_waitcnt vmcnt(0)) before the barrier that publishes the stage.
// `gsrc` is the wave-uniform source of the 1 KB piece (scalar base), `lane_off` = 16 * lane.
__device__ __forceinline__ void copy_1k_to_lds(const char* gsrc, uint32_t lane_off, uint32_t lds_off) {
    lds_off = __builtin_amdgcn_readfirstlane(lds_off);          // wave-uniform by construction; make them scalars
    const uint64_t g = (uint64_t)gsrc;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)g), hi = __builtin_amdgcn_readfirstlane((uint32_t)(g >> 32));
    const uint64_t gs = ((uint64_t)hi << 32) | lo;
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_off), "v"(lane_off), "s"(gs));
}

template <typename T, bool FULL>
__global__ __launch_bounds__(256) void gdn_chunk_wide_kernel(ChunkParams p, SegmentPlan sp) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
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

    const char* Wf = (const char*)p.ws.Wf;
    const char* Uf = (const char*)p.ws.Uf;
    const char* KTf = (const char*)p.ws.KTf;
    const char* Pf = (const char*)p.ws.Pf;
    const char* Qf = (const char*)p.ws.Qf;
    const char* Tab = (const char*)p.ws.Tab;
    T* og = (T*)p.o;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;

    // Every wave copies a quarter of the 1-KB pieces of a stage.  A stage has two parts with
    // separate lifetimes: the operands of the first half of a step (w, u, q, P, tables) and k^T,
    // the operand of the state update in the second half.
    auto copy_first = [&](int64_t it, int stage) {
        const int64_t ci = boh + it;
        const int64_t chv = ci * HV + hv, ch = ci * H + h;
        const uint32_t base = lds0 + stage * STG_BYTES;
        const uint32_t l16 = lane * 16;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int pc = (4 * j + w) * 1024;
            copy_1k_to_lds(Wf + chv * (WS_W * 2) + pc, l16, base + STG_W + pc);
            copy_1k_to_lds(Uf + chv * (WS_U * 2) + pc, l16, base + STG_U + pc);
            if constexpr (FULL) copy_1k_to_lds(Qf + ch * (WS_Q * 2) + pc, l16, base + STG_Q + pc);
        }
        if constexpr (FULL) {
            // P: workspace pieces 0,2,4,5,6,7 (the others are zero); wave w takes slot w, waves 0/1 also slots 4/5
            const int src0 = w < 2 ? 2 * w : w + 2;
            copy_1k_to_lds(Pf + chv * (WS_P * 2) + src0 * 1024, l16, base + STG_P + w * 1024);
            if (w < 2) copy_1k_to_lds(Pf + chv * (WS_P * 2) + (6 + w) * 1024, l16, base + STG_P + (4 + w) * 1024);
        }
        if (w == 0) copy_1k_to_lds(Tab + chv * (WS_TAB * 4), l16, base + STG_TAB);
    };
    auto copy_kt = [&](int64_t it, int stage) {
        const int64_t ch = (boh + it) * H + h;
        const uint32_t base = lds0 + stage * STG_BYTES;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int pc = (4 * j + w) * 1024;
            copy_1k_to_lds(KTf + ch * (WS_KT * 2) + pc, lane * 16, base + STG_KT + pc);
        }
    };
    // A wave issues at least FIRST_MIN copies per copy_first and exactly 4 per copy_kt.  Loads
    // complete in issue order, so "at most FIRST_MIN + 4 operations outstanding" proves that
    // everything older than the last copy_first + copy_kt pair has landed (outstanding stores only
    // make the wait longer).
    auto wait_all_but_newest_pair = [&]() {
        if constexpr (FULL) asm volatile("s_waitcnt vmcnt(17)" ::: "memory");      // 4 w + 4 u + 4 q + 1 P, + 4 k^T
        else asm volatile("s_waitcnt vmcnt(12)" ::: "memory");                     // 4 w + 4 u, + 4 k^T
    };

    const int64_t lastc = it1 - 1;
    if (nsteps > 0) {                         // these travel while the state is loaded
        copy_first(it0, 0);
        copy_kt(it0, 0);
        copy_first(min(it0 + 1, lastc), 1);
    }


    // ---- state: all key rows, value columns 32w .. 32w+31 (tiles n = 2w, 2w+1), C/D layout ----
    f32x4 S[8][2];
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
        for (int nn = 0; nn < 2; ++nn) {
            const int kk = 16 * m + 4 * g, vc = 32 * w + 16 * nn + c16;
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
            if (init == 1) {
#pragma unroll
                for (int r = 0; r < 4; ++r) s[r] = (kk + r == vc) ? 1.f : 0.f;
            } else if (init == 0 && src) {
                if (src_user && vfirst) s = *(const f32x4*)(src + vc * 128 + kk);
                else s = f32x4{src[kk * 128 + vc], src[(kk + 1) * 128 + vc], src[(kk + 2) * 128 + vc], src[(kk + 3) * 128 + vc]};
            }
            S[m][nn] = s;
        }

    // Lazy decay: registers hold S / Gamma, Gamma = 2^lg one scalar per workgroup (see the slab kernel).
    constexpr float LG_MIN = std::is_same<T, bf16_t>::value ? -60.f : 1.f;
    float lg = 0.f;

    // Output: the transposed tiles give each lane 4 consecutive value columns of one token row.
    // They go through this wave's private LDS tile [64 rows][64 B] and leave as 16-byte stores
    // (4 lanes per row, 16 rows per instruction), one step later so that the wait for the stage
    // copies at the end of a step does not also wait for stores issued a moment ago.
    char* otile = smem + 2 * STG_BYTES + w * OT_BYTES;
    auto store_pending = [&](int64_t it) {
        const int valid = (int)min((int64_t)CH, len - it * CH);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int trow = 16 * j + (lane >> 2);
            const u32x4 x = *(const u32x4*)(otile + trow * OT_PITCH + (lane & 3) * 16);
            if (trow < valid) *(u32x4*)(og + ((bos + it * CH + trow) * HV + hv) * 128 + 32 * w + (lane & 3) * 8) = x;
        }
    };

    V8 Vg[2][2];          // v_new decayed to the chunk end, B operand of the state update (first half -> second half)
    auto first_half = [&](int64_t it, const char* st) {
        const V8* sW = (const V8*)(st + STG_W);
        const V8* sQ = (const V8*)(st + STG_Q);
        const V8* sP = (const V8*)(st + STG_P);
        const V4* sU = (const V4*)(st + STG_U);
        const float* sTab = (const float*)(st + STG_TAB);
        // (a) the state as B operand: pairs of key tiles (2s, 2s+1)
        V8 Sb[4][2];
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int nn = 0; nn < 2; ++nn)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    Sb[s][nn][r] = from_f32<T>(S[2 * s][nn][r]);
                    Sb[s][nn][4 + r] = from_f32<T>(S[2 * s + 1][nn][r]);
                }
        const float gamma = fast_exp2(lg);
        const float lg_try = lg + sTab[128];
        const bool lazy = lg_try >= LG_MIN;
        const float vscale = lazy ? fast_exp2(-lg_try) : 1.f;
        V8 Vn[2][2];
        // two t-tiles at a time: w S -> v_new, and the output rows of those tiles
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            f32x4 av[2][2], ao[2][2];
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const int tt = 2 * hf + t2;
#pragma unroll
                for (int nn = 0; nn < 2; ++nn) { av[t2][nn] = f32x4{0.f, 0.f, 0.f, 0.f}; ao[t2][nn] = f32x4{0.f, 0.f, 0.f, 0.f}; }
                V8 aw[4], aq[4];
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    aw[s] = sW[(tt * 4 + s) * 64 + lane];
                    if constexpr (FULL) aq[s] = sQ[(tt * 4 + s) * 64 + lane];
                }
#pragma unroll
                for (int s = 0; s < 4; ++s)
#pragma unroll
                    for (int nn = 0; nn < 2; ++nn) {
                        av[t2][nn] = Mma<T>::run(aw[s], Sb[s][nn], av[t2][nn]);
                        if constexpr (FULL) ao[t2][nn] = Mma<T>::run(Sb[s][nn], aq[s], ao[t2][nn]);   // transposed tile
                    }
            }
            // v_new = u - w S, plain (for the output) and decayed to the chunk end (for the state)
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const int tt = 2 * hf + t2;
                const f32x4 dec = *(const f32x4*)(sTab + 16 * tt + 4 * g) * vscale;
#pragma unroll
                for (int nn = 0; nn < 2; ++nn) {
                    const V4 u4 = sU[((2 * w + nn) * 4 + tt) * 64 + lane];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float uu = u_zero ? 0.f : to_f32(u4[r]);
                        const float vn = uu - gamma * av[t2][nn][r];
                        Vn[hf][nn][t2 * 4 + r] = from_f32<T>(vn);
                        Vg[hf][nn][t2 * 4 + r] = from_f32<T>(vn * dec[r]);
                    }
                }
            }
            // o^T = scale 2^G (q S)^T + (P v_new)^T; each lane stores 4 consecutive value columns of a token row
            if constexpr (FULL) {
#pragma unroll
                for (int t2 = 0; t2 < 2; ++t2) {
                    const int tt = 2 * hf + t2;
                    const float gam = sTab[64 + 16 * tt + c16] * gamma;
                    V8 ap[2];
#pragma unroll
                    for (int sp2 = 0; sp2 <= hf; ++sp2) ap[sp2] = sP[p_slot(tt, sp2) * 64 + lane];
#pragma unroll
                    for (int nn = 0; nn < 2; ++nn) {
                        f32x4 acc = ao[t2][nn] * gam;
#pragma unroll
                        for (int sp2 = 0; sp2 <= hf; ++sp2) acc = Mma<T>::run(Vn[sp2][nn], ap[sp2], acc);
                        V4 o4;
#pragma unroll
                        for (int r = 0; r < 4; ++r) o4[r] = from_f32<T>(acc[r]);
                        *(V4*)(otile + (16 * tt + c16) * OT_PITCH + (16 * nn + 4 * g) * 2) = o4;
                    }
                }
            }
        }
        if (__builtin_amdgcn_readfirstlane((int)lazy) == 0) {       // scalar branch: rare, must not be if-converted
            const float fold = fast_exp2(lg_try);
#pragma unroll
            for (int m = 0; m < 8; ++m)
#pragma unroll
                for (int nn = 0; nn < 2; ++nn) S[m][nn] *= fold;
        }
        lg = lazy ? lg_try : 0.f;
    };
    // S += k^T (v_new decayed)
    auto second_half = [&](const char* st) {
        const V8* sKT = (const V8*)(st + STG_KT);
#pragma unroll
        for (int mh = 0; mh < 4; ++mh) {
            V8 ak[2][2];
#pragma unroll
            for (int mm = 0; mm < 2; ++mm)
#pragma unroll
                for (int sp2 = 0; sp2 < 2; ++sp2) ak[mm][sp2] = sKT[((2 * mh + mm) * 2 + sp2) * 64 + lane];
#pragma unroll
            for (int mm = 0; mm < 2; ++mm)
#pragma unroll
                for (int sp2 = 0; sp2 < 2; ++sp2)
#pragma unroll
                    for (int nn = 0; nn < 2; ++nn)
                        S[2 * mh + mm][nn] = Mma<T>::run(ak[mm][sp2], Vg[sp2][nn], S[2 * mh + mm][nn]);
        }
    };
    if (nsteps > 0) {
        // (the loads of the initial state are older than the copies and complete before them)
        wait_all_but_newest_pair();                             // the first half of stage 0 has landed
        __syncthreads();
        for (int64_t i = 0; i < nsteps; ++i) {
            const int64_t it = it0 + i;
            const int cur = (int)(i & 1);
            char* st = smem + cur * STG_BYTES;
            copy_kt(min(it + 1, lastc), cur ^ 1);               // that k^T region was last read before the previous barrier
            if constexpr (FULL) { if (i > 0) store_pending(it - 1); }
            first_half(it, st);
            wait_all_but_newest_pair();                         // k^T of this chunk has landed ...
            lds_barrier();                                      // ... everywhere, and nobody reads the first-half operands any more
            copy_first(min(it + 2, lastc), cur);
            second_half(st);
            wait_all_but_newest_pair();                         // the first-half operands of the next chunk have landed ...
            lds_barrier();                                      // ... everywhere, and nobody reads this k^T any more
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // no copy may land in LDS after this workgroup has gone
        if constexpr (FULL) store_pending(it1 - 1);
    }

    if (dst) {
        const float gamma = fast_exp2(lg);
#pragma unroll
        for (int m = 0; m < 8; ++m)
#pragma unroll
            for (int nn = 0; nn < 2; ++nn) {
                const int kk = 16 * m + 4 * g, vc = 32 * w + 16 * nn + c16;
                const f32x4 s = S[m][nn] * gamma;
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
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), WIDE_SMEM, stream, p, sp);
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
