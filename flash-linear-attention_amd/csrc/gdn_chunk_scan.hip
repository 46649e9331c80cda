// Sequential stage of the chunked prefill, "slab" form: one workgroup per (sequence, v-head,
// slab of 16*NV value columns) walks the chunks in order with the fp32 state S[K, slab] in
// registers:
//   v_new = u - w S;  o = scale*((q S)*2^G) + P v_new;  S = 2^G_last S + k^T (v_new*2^(G_last-G)).
// Per-chunk states and v_new never go to memory.  Used when there are too few (sequence,
// head) pairs to give every CU a whole head.
#include "gdn_chunk_common.h"

namespace gdn {

template <typename T, int NV>
struct ScanFrags {
    typename Mma<T>::V8 wf[4], qf[4], kt[2][2], pf[2];
    typename Mma<T>::V4 uf[NV];
    f32x4 dec;          // 2^(G_last-G_t) for the 4 rows of this lane's C/D fragment
    float gam;          // scale*2^G_t for the column of this lane's transposed output fragment
    float glast;        // G_last in log2 units
    int valid;
};

template <typename T, int NV>
__global__ __launch_bounds__(256) void gdn_chunk_scan_kernel(ChunkParams p) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    extern __shared__ __align__(16) char smem[];
    V8* sSb = (V8*)smem;                    // [4 s][NV][64] state as B operand (key tiles 2s, 2s+1)
    V4* sVn = (V4*)(sSb + 4 * NV * 64);     // [2 kind][2 s][NV][64][2 half] v_new as B operand (t-tiles 2s, 2s+1)

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, g = lane >> 4;
    // Workgroups are dealt to the 8 XCDs round-robin by block index; keep all slabs of one
    // (sequence, head) on one XCD so that they share w / k^T / P / q through that XCD's L2.
    const int xcd = blockIdx.x & 7;
    const int64_t y = blockIdx.x >> 3;
    const int64_t inh = xcd + 8 * (y / p.nslab);
    const int slab = (int)(y % p.nslab);
    if (inh >= p.NH) return;
    const int H = p.H, HV = p.HV;
    const int64_t n = inh / HV;
    const int hv = (int)(inh % HV);
    const int h = hv / (HV / H);
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    const bool vfirst = p.flags & GDN_FLAG_STATE_V_FIRST;

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
    const int v0 = slab * NV * 16;          // first value column of this slab

    // ---- state: this wave owns key tiles 2w, 2w+1 (rows 32w .. 32w+31), C/D layout ----
    f32x4 S[2][NV];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
            if (p.h0) {
                const int kk = 32 * w + 16 * i + 4 * g, vc = v0 + 16 * nn + c16;
                const float* base = p.h0 + inh * 128 * 128;
                if (vfirst) s = *(const f32x4*)(base + vc * 128 + kk);
                else s = f32x4{base[kk * 128 + vc], base[(kk + 1) * 128 + vc], base[(kk + 2) * 128 + vc], base[(kk + 3) * 128 + vc]};
            }
            S[i][nn] = s;
        }

    // Make the initial state arrive before the prefetch queue is started: a wait for these
    // registers inside the loop (their first use) would be executed on every trip and would
    // drain the prefetched loads with it.
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) asm volatile("" : "+v"(S[i][nn]) : : "memory");

    const T* Wf = (const T*)p.ws.Wf;
    const T* Uf = (const T*)p.ws.Uf;
    const T* KTf = (const T*)p.ws.KTf;
    const T* Pf = (const T*)p.ws.Pf;
    const T* Qf = (const T*)p.ws.Qf;
    T* og = (T*)p.o;

    // All loads are unconditional and there is no data-dependent control flow around memory
    // operations in the main loop: the compiler can then count outstanding loads exactly and
    // wait only for the buffer it is about to use, instead of draining the queue.
    auto load_a = [&](int64_t it, ScanFrags<T, NV>& f) {        // operands of the first half of a step
        const int64_t ci = boh + it;
        const int64_t chv = ci * HV + hv, ch = ci * H + h;
#pragma unroll
        for (int s = 0; s < 4; ++s) f.wf[s] = *(const V8*)(Wf + chv * WS_W + ((w * 4 + s) * 64 + lane) * 8);
#pragma unroll
        for (int s = 0; s < 4; ++s) f.qf[s] = *(const V8*)(Qf + ch * WS_Q + ((w * 4 + s) * 64 + lane) * 8);
    };
    auto load_b = [&](int64_t it, ScanFrags<T, NV>& f) {        // everything else
        const int64_t ci = boh + it;
        const int64_t chv = ci * HV + hv, ch = ci * H + h;
        f.valid = (int)min((int64_t)CH, len - it * CH);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int s = 0; s < 2; ++s)
                f.kt[i][s] = *(const V8*)(KTf + ch * WS_KT + (((2 * w + i) * 2 + s) * 64 + lane) * 8);
#pragma unroll
        for (int s = 0; s < 2; ++s) f.pf[s] = *(const V8*)(Pf + chv * WS_P + ((w * 2 + s) * 64 + lane) * 8);
#pragma unroll
        for (int nn = 0; nn < NV; ++nn)
            f.uf[nn] = *(const V4*)(Uf + chv * WS_U + (((v0 / 16 + nn) * 4 + w) * 64 + lane) * 4);
        const float* tab = p.ws.Tab + chv * WS_TAB;
        f.dec = *(const f32x4*)(tab + 16 * w + 4 * g);
        f.gam = tab[64 + 16 * w + c16];
        f.glast = tab[128];
    };

    // The registers hold Shat = S / Gamma with one scalar Gamma = 2^lg per workgroup, so the
    // decay of the whole state by 2^G_last per chunk costs nothing: products with S are
    // rescaled by Gamma (folded into multiplies that exist anyway) and the update is divided
    // by the new Gamma (folded into the decay factors of v_new).  When Gamma gets small the
    // state is rescaled once and Gamma restarts at 1.  f16 operands have too little range for
    // Shat, so there the state is rescaled on every chunk.
    constexpr float LG_MIN = std::is_same<T, bf16_t>::value ? -60.f : 1.f;
    float lg = 0.f;                                              // log2 Gamma

    // `f` holds the chunk being processed; `fr` is the buffer consumed one step earlier, which is
    // refilled with chunk `refill` while this step computes (its loads are interleaved with the
    // matrix instructions so that the memory pipeline never sees a burst).
    auto step = [&](int64_t it, ScanFrags<T, NV>& f, ScanFrags<T, NV>& fr, int64_t refill, auto masked) {
        // (a) publish the state at the start of this chunk as bf16/f16 B-operand fragments
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            V8 sb;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sb[r] = from_f32<T>(S[0][nn][r]);
                sb[4 + r] = from_f32<T>(S[1][nn][r]);
            }
            sSb[(w * NV + nn) * 64 + lane] = sb;
        }
        const float gamma = fast_exp2(lg);
        const float lg_try = lg + f.glast;
        const bool lazy = lg_try >= LG_MIN;                      // same value in every lane of the workgroup
        const float vscale = lazy ? fast_exp2(-lg_try) : 1.f;
        const f32x4 dec = f.dec * vscale;
        const float ogam = f.gam * gamma;
        lds_barrier();
        // (b,c) w S (rows of t-tile w) and (q S)^T (columns of t-tile w)
        f32x4 acco[NV];
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            f32x4 av = {0.f, 0.f, 0.f, 0.f}, ao = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const V8 sb = sSb[(s * NV + nn) * 64 + lane];
                av = Mma<T>::run(f.wf[s], sb, av);
                ao = Mma<T>::run(sb, f.qf[s], ao);      // operands swapped: result is the transposed tile
            }
            acco[nn] = ao * ogam;
            // (d) v_new = u - w S; publish it plain (for the output) and decayed to the chunk end (for the state)
            V4 plain, gated;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float vn = to_f32(f.uf[nn][r]) - gamma * av[r];
                plain[r] = from_f32<T>(vn);
                gated[r] = from_f32<T>(vn * dec[r]);
            }
            sVn[(((0 * 2 + (w >> 1)) * NV + nn) * 64 + lane) * 2 + (w & 1)] = plain;
            sVn[(((1 * 2 + (w >> 1)) * NV + nn) * 64 + lane) * 2 + (w & 1)] = gated;
        }
        if (!decltype(masked)::value) {
            load_a(refill, fr);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                __builtin_amdgcn_sched_group_barrier(0x008, NV, 0);      // NV matrix instructions
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);       // then one global load
            }
        }
        if (__builtin_amdgcn_readfirstlane((int)lazy) == 0) {       // scalar branch: rare, must not be if-converted
            const float fold = fast_exp2(lg_try);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int nn = 0; nn < NV; ++nn) S[i][nn] *= fold;
        }
        lg = lazy ? lg_try : 0.f;
        lds_barrier();
        // (e,f) state update and output
        const V8* sVn8 = (const V8*)sVn;
        const int trow = 16 * w + c16;
        T* orow = og + ((bos + it * CH + trow) * HV + hv) * 128 + v0 + 4 * g;
#pragma unroll
        for (int nn = 0; nn < NV; ++nn) {
            const V8 vg0 = sVn8[((1 * 2 + 0) * NV + nn) * 64 + lane], vg1 = sVn8[((1 * 2 + 1) * NV + nn) * 64 + lane];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                f32x4 s = S[i][nn];
                s = Mma<T>::run(f.kt[i][0], vg0, s);
                s = Mma<T>::run(f.kt[i][1], vg1, s);
                S[i][nn] = s;
            }
            // P rows of t-tile w reach t-tiles <= w only; the fragments above the diagonal are zero
            f32x4 ao = Mma<T>::run(sVn8[((0 * 2 + 0) * NV + nn) * 64 + lane], f.pf[0], acco[nn]);
            ao = Mma<T>::run(sVn8[((0 * 2 + 1) * NV + nn) * 64 + lane], f.pf[1], ao);
            // transposed tile: this lane holds 4 consecutive value columns of token row trow
            V4 o4;
#pragma unroll
            for (int r = 0; r < 4; ++r) o4[r] = from_f32<T>(ao[r]);
            if (!decltype(masked)::value) store_b64_uncounted(orow + 16 * nn, __builtin_bit_cast(u32x2, o4));
            else if (trow < f.valid) *(V4*)(orow + 16 * nn) = o4;
        }
        if (!decltype(masked)::value) {
            load_b(refill, fr);
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                __builtin_amdgcn_sched_group_barrier(0x008, NV, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
            }
        }
    };
    std::integral_constant<bool, false> full_chunk;
    std::integral_constant<bool, true> tail_chunk;

    // NB fragment buffers in rotation: step `it` computes from buffer it%NB and refills buffer
    // (it-1)%NB (consumed in the previous step) with chunk it+NB-1, so every load has NB-2 full
    // steps to arrive.  A wave can have 63 loads in flight, 18 per buffer, hence NB = 4.
    // Refills past the end re-read the last chunk and are never used.
    constexpr int NB = NV >= 8 ? 3 : 4;          // the widest slab has no registers to spare and is compute-bound anyway
    ScanFrags<T, NV> fb[NB];
    const int64_t last = nt - 1;
    const int64_t nfast = (len / CH) / NB * NB;     // chunks handled NB at a time; all of them are full
    if (nt > 0) {
        // compiler fences keep the groups in issue order, as inside the loop: the waits in the
        // loop are sized for the entry path too
#pragma unroll
        for (int j = 0; j < NB - 1; ++j) {
            load_a(min((int64_t)j, last), fb[j]);
            asm volatile("" ::: "memory");
            load_b(min((int64_t)j, last), fb[j]);
            asm volatile("" ::: "memory");
        }
    }
    for (int64_t it = 0; it < nfast; it += NB) {
#pragma unroll
        for (int j = 0; j < NB; ++j) step(it + j, fb[j], fb[(j + NB - 1) % NB], min(it + j + NB - 1, last), full_chunk);
    }
    // at most NB chunks remain (NB-1 full ones and a ragged tail): buffers 0..NB-2 already hold
    // the first of them
    if (nfast + NB - 1 < nt) {
        load_a(nfast + NB - 1, fb[NB - 1]);
        load_b(nfast + NB - 1, fb[NB - 1]);
    }
#pragma unroll
    for (int j = 0; j < NB; ++j)
        if (nfast + j < nt) step(nfast + j, fb[j], fb[j], 0, tail_chunk);

    // back to the true state
    {
        const float gamma = fast_exp2(lg);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int nn = 0; nn < NV; ++nn) S[i][nn] *= gamma;
    }

    if (p.ht) {
        float* base = p.ht + inh * 128 * 128;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int nn = 0; nn < NV; ++nn) {
                const int kk = 32 * w + 16 * i + 4 * g, vc = v0 + 16 * nn + c16;
                if (vfirst) *(f32x4*)(base + vc * 128 + kk) = S[i][nn];
                else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) base[(kk + r) * 128 + vc] = S[i][nn][r];
                }
            }
    }
}

template <typename T, int NV>
static int launch_scan_nv(const ChunkParams& p0, hipStream_t stream) {
    ChunkParams p = p0;
    p.nslab = 8 / NV;
    const size_t smem = (size_t)4 * NV * 64 * 16 + (size_t)2 * 2 * NV * 64 * 16;
    auto kern = gdn_chunk_scan_kernel<T, NV>;
    if (smem > 48 * 1024) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
            return check_launch("hipFuncSetAttribute(scan)");
    }
    const int64_t groups = (p.NH + 7) / 8;
    dim3 grid((unsigned)(groups * 8 * p.nslab)), block(256);
    hipLaunchKernelGGL(kern, grid, block, smem, stream, p);
    return check_launch("gdn_chunk_scan_kernel");
}

template <typename T>
int launch_scan_slab(const ChunkParams& p, hipStream_t stream) {
    // widest value slab that still gives every CU a workgroup
    if (p.NH >= 256) return launch_scan_nv<T, 8>(p, stream);
    if (p.NH * 2 >= 256) return launch_scan_nv<T, 4>(p, stream);
    if (p.NH * 4 >= 256) return launch_scan_nv<T, 2>(p, stream);
    return launch_scan_nv<T, 1>(p, stream);
}
template int launch_scan_slab<bf16_t>(const ChunkParams&, hipStream_t);
template int launch_scan_slab<f16_t>(const ChunkParams&, hipStream_t);

}  // namespace gdn
