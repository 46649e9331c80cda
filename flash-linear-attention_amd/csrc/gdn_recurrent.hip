// Token recurrence of the gated delta rule (decode and short prompts) for gfx950.
//
//   S <- e^{g_t} S (and e^{gk}, e^{gv});  d = beta_t (v_t - S^T k_t);  S <- S + k_t d^T;  o_t = scale S^T q_t
//
// One workgroup of 256 threads owns the state of one (sequence, v-head) restricted to a
// block of VB value columns (K-first layout [K,V]) or VB value rows (V-first layout
// [V,K]).  The fp32 state lives in registers for the whole call: each thread holds R
// float4 pieces, every global access is a 16-byte piece of a contiguous row, so one wave
// instruction reads whole rows - the step is a pure HBM stream of the state (read once,
// written once, in place if the caller aliases ht to h0).
//
// The comba operator (fla/ops/comba/fused_recurrent.py:85-105) is the same recurrence with a second key p for the
// prediction, taken on the state BEFORE the token's decay:  d = beta_t (v_t - S^T p_t);  S <- e^{g_t} S + k_t d^T.
#include "gdn_common.h"

namespace gdn {

struct RecurrentParams {
    const void* q; const void* k; const void* v;
    const void* pk;                      // comba: the key the prediction is made with (NULL otherwise)
    const void* g; const void* beta; const float* gk; const float* gv;
    const float* A_log; const float* dt_bias;
    const float* h0; float* ht; void* o;
    const void* cu_seqlens; const void* state_slots; const void* num_accepted;
    int64_t slots_stride;
    int64_t T; int H, HV, K, V, NVB;
    float scale; int gb_dtype; uint32_t flags;
    int xcd_group; int64_t nblocks;      // see xcd_block()
    // gate per key feature given as a raw input (the KDA operator): 0 = gk is the log decay itself,
    // 1: gk <- -e^A softplus(gk + bias), 2: gk <- lower sigmoid(e^A (gk + bias)); A = A_log[head] (mode 1 without
    // A_log: A = 1, mode 2 without: e^A = 1), bias = gk_bias[head][key feature] or 0
    int gk_act; const float* gk_bias; float gk_lower;
};

// log decay of key feature `kidx` for token `tok` (see RecurrentParams::gk_act)
__device__ __forceinline__ float gate_k(const RecurrentParams& p, int64_t tok, int ihv, int kidx, float a_k) {
    float x = p.gk[(tok * p.HV + ihv) * p.K + kidx];
    if (p.gk_act) {
        if (p.gk_bias) x += p.gk_bias[ihv * p.K + kidx];
        x = p.gk_act == 2 ? p.gk_lower * sigmoid_f(a_k * x) : -a_k * softplus_f(x);
    }
    return x;
}

// Workgroups are dealt to the chip's 8 XCDs round-robin by block index.  With xcd_group = g > 0 the work items (state
// blocks, consecutive in memory) are handed out so that every XCD works on runs of g consecutive items instead of
// every eighth one: an XCD then touches an eighth of the pages the launch touches, not all of them.  The grid is
// rounded up to whole rounds of 8 groups; -1 = nothing to do for this workgroup.
__device__ __forceinline__ int64_t xcd_block(const RecurrentParams& p) {
    int64_t blk = blockIdx.x;
    if (p.xcd_group > 0) {
        const int64_t s = blk >> 3;
        blk = ((s / p.xcd_group) * 8 + (blk & 7)) * p.xcd_group + s % p.xcd_group;
        if (blk >= p.nblocks) return -1;
    }
    return blk;
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// KMAX: compile-time bound on K (rows padded with zeros), VB: value block per workgroup.
template <typename T, int KMAX, int VB, bool VFIRST, bool COMBA = false>
__global__ __launch_bounds__(256) void gdn_recurrent_kernel(RecurrentParams p) {
    static_assert(!(COMBA && VFIRST), "the comba recurrence is built for the K-first layout");
    // lanes along the contiguous dim (float4 each), the rest of the 256 threads along rows
    constexpr int CONT = VFIRST ? KMAX : VB;        // extent of the contiguous dim handled
    constexpr int TC = CONT / 4;                    // threads along the contiguous dim
    constexpr int RP = 256 / TC;                    // rows per pass
    constexpr int ROWS = VFIRST ? VB : KMAX;        // extent of the row dim handled
    constexpr int R = (ROWS + RP - 1) / RP;         // float4 pieces per thread
    static_assert(TC <= 64 && (TC & (TC - 1)) == 0, "contiguous extent must map to <= 64 lanes");

    const int tid = threadIdx.x;
    const int c = tid % TC, r0 = tid / TC;
    const int wave = tid >> 6;
    const int64_t blk = xcd_block(p);
    if (blk < 0) return;
    const int ivb = (int)(blk % p.NVB);
    const int64_t inh = blk / p.NVB;
    const int64_t in = inh / p.HV;
    const int ihv = (int)(inh % p.HV);
    const int ih = ihv / (p.HV / p.H);
    const int K = p.K, V = p.V, H = p.H, HV = p.HV;
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;

    int64_t bos, len;
    if (p.cu_seqlens) {
        bos = load_index(p.cu_seqlens, in, cu32);
        len = load_index(p.cu_seqlens, in + 1, cu32) - bos;
    } else {
        bos = in * p.T;
        len = p.T;
    }
    const int v0 = ivb * VB;                        // first value index of this block

    // ---- state into registers (issued first: everything else hides behind these loads) ----
    f32x4 S[R];
    // K-first: row = k index, cont = v index.  V-first: row = v index, cont = k index.
    const int cont_idx = (VFIRST ? 0 : v0) + 4 * c;
    const int cont_lim = VFIRST ? K : V;
    const int row_lim = VFIRST ? V : K;
    const int row_base = VFIRST ? v0 : 0;
    const int64_t row_stride = VFIRST ? K : V;
    const bool cont_ok = cont_idx < cont_lim;
    // The state lives at sequence n of the state tensors, or at the slot of a pool that the caller names for n.
    // With a slot per token (speculative decoding) the sequence starts from the slot of its last accepted token
    // (the first one without num_accepted) and leaves the state after token t in slot (n, t).
    const bool slot32 = p.flags & GDN_FLAG_SLOT_INT32;
    const bool slot_per_token = p.flags & GDN_FLAG_SLOT_PER_TOKEN, state_per_token = p.flags & GDN_FLAG_STATE_PER_TOKEN;
    int64_t slot = in;
    if (p.state_slots) {
        int64_t first = 0;
        // (a count outside 1 .. row width would index past this sequence's row of the table: held to the row)
        if (slot_per_token && p.num_accepted)
            first = min(max(load_index(p.num_accepted, in, slot32) - 1, (int64_t)0), p.slots_stride - 1);
        slot = load_index(p.state_slots, slot_per_token ? in * p.slots_stride + first : in, slot32);
    }
    const int64_t head_off = (int64_t)ihv * K * V, state_stride = (int64_t)HV * K * V;
    const int64_t state_off = slot * state_stride + head_off;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int row = row_base + r0 + RP * i;
        const bool ok = cont_ok && (r0 + RP * i < ROWS) && row < row_lim;
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        if (ok && p.h0) s = __builtin_nontemporal_load((const f32x4*)(p.h0 + state_off + row * row_stride + cont_idx));
        S[i] = s;
    }

    auto store_state = [&](float* dst) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int row = row_base + r0 + RP * i;
            const bool ok = cont_ok && (r0 + RP * i < ROWS) && row < row_lim;
            if (ok) __builtin_nontemporal_store(S[i], (f32x4*)(dst + row * row_stride + cont_idx));
        }
    };

    __shared__ float sh_q[2][KMAX], sh_k[2][KMAX], sh_p[2][COMBA ? KMAX : 1];
    __shared__ float sh_red[2][4][4];                       // per-wave partial sums for |q|^2, |k|^2, q.k, |p|^2
    __shared__ float sh_part[2][4][2][VFIRST ? 4 : VB];     // K-first: per-wave column sums for S^T k and S^T q

    const T* q = (const T*)p.q; const T* k = (const T*)p.k; const T* v = (const T*)p.v; T* o = (T*)p.o;
    float a_neg = 0.f, dtb = 0.f;
    if (p.A_log && !p.gk_act) { a_neg = -__expf(p.A_log[ihv]); if (p.dt_bias) dtb = p.dt_bias[ihv]; }
    const float a_k = p.gk_act ? (p.A_log ? __expf(p.A_log[ihv]) : (p.gk_act == 2 ? 1.f : __expf(1.f))) : 0.f;

    for (int64_t t = 0; t < len; ++t) {
        const int pb = (int)(t & 1);
        const int64_t tok = bos + t;
        // -- stage q_t, k_t and their three inner products
        float qv = 0.f, kv = 0.f;
        if (tid < K) {
            qv = to_f32(q[(tok * H + ih) * K + tid]);
            kv = to_f32(k[(tok * H + ih) * K + tid]);
        }
        if (tid < KMAX) { sh_q[pb][tid] = qv; sh_k[pb][tid] = kv; }
        float sqq = wave_sum(qv * qv), skk = wave_sum(kv * kv), sqk = wave_sum(qv * kv);
        if ((tid & 63) == 0) { sh_red[pb][wave][0] = sqq; sh_red[pb][wave][1] = skk; sh_red[pb][wave][2] = sqk; }
        if constexpr (COMBA) {
            const float pv = tid < K ? to_f32(((const T*)p.pk)[(tok * H + ih) * K + tid]) : 0.f;
            if (tid < KMAX) sh_p[pb][tid] = pv;
            const float spp = wave_sum(pv * pv);
            if ((tid & 63) == 0) sh_red[pb][wave][3] = spp;
        }
        // per-token scalars / per-column vectors (independent of the state)
        float eg = 1.f;
        if (p.g) {
            float gt = load_scalar(p.g, tok * HV + ihv, p.gb_dtype);
            if (p.A_log && !p.gk_act) gt = a_neg * softplus_f(gt + dtb);
            eg = __expf(gt);
        }
        __syncthreads();
        sqq = sh_red[pb][0][0] + sh_red[pb][1][0] + sh_red[pb][2][0] + sh_red[pb][3][0];
        skk = sh_red[pb][0][1] + sh_red[pb][1][1] + sh_red[pb][2][1] + sh_red[pb][3][1];
        sqk = sh_red[pb][0][2] + sh_red[pb][1][2] + sh_red[pb][2][2] + sh_red[pb][3][2];
        float rq = p.scale, rk = 1.f, rp = 1.f;
        if (p.flags & GDN_FLAG_QK_L2NORM) {
            rq *= 1.f / sqrtf(sqq + 1e-6f);
            rk = 1.f / sqrtf(skk + 1e-6f);
            if constexpr (COMBA) rp = 1.f / sqrtf(sh_red[pb][0][3] + sh_red[pb][1][3] + sh_red[pb][2][3] + sh_red[pb][3][3] + 1e-6f);
        }
        const float qk = sqk * rq * rk;             // (scale q).k after normalisation

        if constexpr (!VFIRST) {
            // ---------------- K-first: rows are k, this thread owns 4 value columns ----------------
            float kr[R], qr[R], pr[COMBA ? R : 1];
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const int row = r0 + RP * i;
                kr[i] = row < KMAX ? sh_k[pb][row] * rk : 0.f;
                qr[i] = row < KMAX ? sh_q[pb][row] * rq : 0.f;
                if constexpr (COMBA) pr[i] = row < KMAX ? sh_p[pb][row] * rp : 0.f;
            }
            f32x4 dgv = {1.f, 1.f, 1.f, 1.f};
            if (p.gv && cont_ok) {
                const f32x4 x = *(const f32x4*)(p.gv + (tok * HV + ihv) * V + cont_idx);
                dgv = f32x4{__expf(x.x), __expf(x.y), __expf(x.z), __expf(x.w)};
            }
            dgv *= eg;
            f32x4 sk = {0.f, 0.f, 0.f, 0.f}, sq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < R; ++i) {
                if constexpr (COMBA) sk += S[i] * pr[i];     // the prediction sees the state before this token's decay
                f32x4 s = S[i] * dgv;
                if (p.gk) {
                    const int row = r0 + RP * i;
                    if (row < K) s *= __expf(gate_k(p, tok, ihv, row, a_k));
                }
                S[i] = s;
                if constexpr (!COMBA) sk += s * kr[i];
                sq += s * qr[i];
            }
            // reduce over the row groups that share this thread's columns: inside the wave, then across waves
#pragma unroll
            for (int off = TC; off < 64; off <<= 1) {
#pragma unroll
                for (int j = 0; j < 4; ++j) { sk[j] += __shfl_xor(sk[j], off, 64); sq[j] += __shfl_xor(sq[j], off, 64); }
            }
            if ((tid & 63) < TC) {
                *(f32x4*)&sh_part[pb][wave][0][4 * c] = sk;
                *(f32x4*)&sh_part[pb][wave][1][4 * c] = sq;
            }
            __syncthreads();
            sk = *(f32x4*)&sh_part[pb][0][0][4 * c] + *(f32x4*)&sh_part[pb][1][0][4 * c] +
                 *(f32x4*)&sh_part[pb][2][0][4 * c] + *(f32x4*)&sh_part[pb][3][0][4 * c];
            sq = *(f32x4*)&sh_part[pb][0][1][4 * c] + *(f32x4*)&sh_part[pb][1][1][4 * c] +
                 *(f32x4*)&sh_part[pb][2][1][4 * c] + *(f32x4*)&sh_part[pb][3][1][4 * c];
            f32x4 vv = {0.f, 0.f, 0.f, 0.f}, bb = {1.f, 1.f, 1.f, 1.f};
            if (cont_ok) {
                const T* pv = v + (tok * HV + ihv) * V + cont_idx;
                vv = f32x4{to_f32(pv[0]), to_f32(pv[1]), to_f32(pv[2]), to_f32(pv[3])};
                // (a missing beta counts as ones BEFORE the activation, fla/ops/gated_delta_rule/fused_recurrent.py:443)
                if (p.beta) {
                    if (p.flags & GDN_FLAG_BETA_VECTOR) {
                        const int64_t bi = (tok * HV + ihv) * V + cont_idx;
                        bb = f32x4{load_scalar(p.beta, bi, p.gb_dtype), load_scalar(p.beta, bi + 1, p.gb_dtype),
                                   load_scalar(p.beta, bi + 2, p.gb_dtype), load_scalar(p.beta, bi + 3, p.gb_dtype)};
                    } else {
                        const float b = load_scalar(p.beta, tok * HV + ihv, p.gb_dtype);
                        bb = f32x4{b, b, b, b};
                    }
                }
                if (p.flags & GDN_FLAG_BETA_SIGMOID) {
                    const float m = (p.flags & GDN_FLAG_NEG_EIGVAL) ? 2.f : 1.f;
                    bb = f32x4{m * sigmoid_f(bb.x), m * sigmoid_f(bb.y), m * sigmoid_f(bb.z), m * sigmoid_f(bb.w)};
                }
            }
            const f32x4 d = bb * (vv - sk);
#pragma unroll
            for (int i = 0; i < R; ++i) S[i] += d * kr[i];
            if (r0 == 0 && cont_ok) {
                const f32x4 ov = sq + d * qk;
                T* po = o + (tok * HV + ihv) * V + cont_idx;
                po[0] = from_f32<T>(ov.x); po[1] = from_f32<T>(ov.y); po[2] = from_f32<T>(ov.z); po[3] = from_f32<T>(ov.w);
            }
        } else {
            // ---------------- V-first: rows are v, this thread owns 4 key columns ----------------
            f32x4 kc = {0.f, 0.f, 0.f, 0.f}, qc = {0.f, 0.f, 0.f, 0.f};
            kc = *(f32x4*)&sh_k[pb][4 * c] * rk;
            qc = *(f32x4*)&sh_q[pb][4 * c] * rq;
            f32x4 dgk = {eg, eg, eg, eg};
            if (p.gk && cont_ok) {
                f32x4 x = *(const f32x4*)(p.gk + (tok * HV + ihv) * K + cont_idx);
                if (p.gk_act) x = f32x4{gate_k(p, tok, ihv, cont_idx, a_k), gate_k(p, tok, ihv, cont_idx + 1, a_k),
                                        gate_k(p, tok, ihv, cont_idx + 2, a_k), gate_k(p, tok, ihv, cont_idx + 3, a_k)};
                dgk *= f32x4{__expf(x.x), __expf(x.y), __expf(x.z), __expf(x.w)};
            }
            const float bmul = (p.flags & GDN_FLAG_NEG_EIGVAL) ? 2.f : 1.f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const int row = v0 + r0 + RP * i;
                const bool rok = (r0 + RP * i < ROWS) && row < V;
                f32x4 s = S[i] * dgk;
                if (p.gv && rok) s *= __expf(p.gv[(tok * HV + ihv) * V + row]);
                f32x4 a = s * kc, b = s * qc;
                float sk = a.x + a.y + a.z + a.w, sq = b.x + b.y + b.z + b.w;
#pragma unroll
                for (int off = 1; off < TC; off <<= 1) { sk += __shfl_xor(sk, off, 64); sq += __shfl_xor(sq, off, 64); }
                float vv = 0.f, bb = 1.f;
                if (rok) {
                    vv = to_f32(v[(tok * HV + ihv) * V + row]);
                    if (p.beta) {
                        bb = (p.flags & GDN_FLAG_BETA_VECTOR) ? load_scalar(p.beta, (tok * HV + ihv) * V + row, p.gb_dtype)
                                                              : load_scalar(p.beta, tok * HV + ihv, p.gb_dtype);
                    }
                    if (p.flags & GDN_FLAG_BETA_SIGMOID) bb = bmul * sigmoid_f(bb);
                }
                const float d = bb * (vv - sk);
                S[i] = s + kc * d;
                if (c == 0 && rok) o[(tok * HV + ihv) * V + row] = from_f32<T>(sq + d * qk);
            }
        }
        // a state per token: into the slot named for (n, t), or into entry `tok` of a per-token state tensor
        // (a token past the row width of the slot table has no slot: its state is kept in registers and not stored)
        if (p.ht && (state_per_token || (slot_per_token && t < p.slots_stride))) {
            const int64_t dst = state_per_token ? tok : load_index(p.state_slots, in * p.slots_stride + t, slot32);
            store_state(p.ht + dst * state_stride + head_off);
        }
    }

    if (p.ht && !slot_per_token && !state_per_token) store_state(p.ht + state_off);
}


// The common decode shape on its own: K = V = 128, K-first states [K][V], one gate and one beta per head, states
// per sequence or per slot.  Same arithmetic as gdn_recurrent_kernel with the decay e^g applied after the reductions,
//   S' = e^g S + k d^T,   d = beta (v - e^g S^T k),   o = scale (e^g S^T q + (q.k) d),
// k and q of a token read from LDS where they are used instead of being held per row.  The token's own rows (q, k,
// v, gate, beta) are requested BEFORE the state: loads return in issue order, so their norms and the LDS staging are
// done while the 64 KB of state are still on their way, and what follows the state's arrival is only the two
// reductions and the update.  Thread (c = tid % 32, r0 = tid / 32) owns value columns 4c .. 4c+3 of key rows r0 + 8i.
// Launched with enough unused LDS that two workgroups share a CU: more resident workgroups widen the window of
// memory the chip works on at one time, and the read-modify-write stream gets slower (measured: 1, 2, 3+ workgroups
// per CU = 208, 183, 191 us for 1 GiB of state traffic).
constexpr size_t DECODE_LDS_PAD = 64 * 1024;

// GK: a decay per key feature as well (the KDA operator's decode step): S' = diag(e^gk) e^g S + k d^T, so the two
// reductions run over e^gk k and e^gk q, staged beside k and q, and the update takes a factor per row.
// PK: a second key p that the prediction uses on the state as it was BEFORE this token's decay (the comba operator's
// decode step): d = beta (v - S^T p), so that reduction runs over p and takes no e^g.
template <typename T, bool GK = false, bool PK = false>
__global__ __launch_bounds__(256, 2) void gdn_decode_kernel(RecurrentParams p) {
    static_assert(!(GK && PK), "one of the two forms at a time");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = tid & 31, r0 = tid >> 5;
    const int64_t inh = xcd_block(p);
    if (inh < 0) return;
    const int64_t in = inh / p.HV;
    const int ihv = (int)(inh % p.HV);
    const int H = p.H, HV = p.HV;
    const int ih = ihv / (HV / H);
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    int64_t bos, len;
    if (p.cu_seqlens) {
        bos = load_index(p.cu_seqlens, in, cu32);
        len = load_index(p.cu_seqlens, in + 1, cu32) - bos;
    } else {
        bos = in * p.T;
        len = p.T;
    }
    const int64_t slot = p.state_slots ? load_index(p.state_slots, in, p.flags & GDN_FLAG_SLOT_INT32) : in;
    const int64_t state_off = (slot * HV + ihv) * (int64_t)16384 + 4 * c;
    const T* q = (const T*)p.q; const T* k = (const T*)p.k; const T* v = (const T*)p.v; T* o = (T*)p.o;
    // what a token brings, as it comes from memory
    struct Token { T q, k, pk; T v[4]; float g, b, gk; };
    const float a_k = GK && p.gk_act ? (p.A_log ? __expf(p.A_log[ihv]) : (p.gk_act == 2 ? 1.f : __expf(1.f))) : 0.f;
    const float gk_bias = GK && p.gk_act && p.gk_bias && tid < 128 ? p.gk_bias[ihv * 128 + tid] : 0.f;
    auto fetch = [&](int64_t tok) {
        Token x;
        x.q = x.k = x.pk = from_f32<T>(0.f);
        x.gk = 0.f;
        if (tid < 128) {
            x.q = q[(tok * H + ih) * 128 + tid]; x.k = k[(tok * H + ih) * 128 + tid];
            if constexpr (GK) x.gk = p.gk[(tok * HV + ihv) * 128 + tid];
            if constexpr (PK) x.pk = ((const T*)p.pk)[(tok * H + ih) * 128 + tid];
        }
        const T* pv = v + (tok * HV + ihv) * 128 + 4 * c;
#pragma unroll
        for (int j = 0; j < 4; ++j) x.v[j] = pv[j];
        x.g = p.g ? load_scalar(p.g, tok * HV + ihv, p.gb_dtype) : 0.f;
        x.b = p.beta ? load_scalar(p.beta, tok * HV + ihv, p.gb_dtype) : 1.f;
        return x;
    };
    Token cur = {};
    if (len > 0) cur = fetch(bos);
    float a_neg = 0.f, dtb = 0.f;
    if (p.A_log) { a_neg = -__expf(p.A_log[ihv]); if (p.dt_bias) dtb = p.dt_bias[ihv]; }
    // ---- the state: 16 requests of 16 bytes per thread, a wave instruction covers two whole rows ----
    f32x4 S[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        S[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (p.h0) S[i] = __builtin_nontemporal_load((const f32x4*)(p.h0 + state_off + (r0 + 8 * i) * 128));
    }
    __shared__ float sh_q[2][128], sh_k[2][128];
    __shared__ float sh_kr[GK ? 2 : 1][GK ? 128 : 1], sh_eg[GK ? 2 : 1][GK ? 128 : 1];     // (GK) k as it is, and e^gk per row
    __shared__ float sh_p[PK ? 2 : 1][PK ? 128 : 1];
    __shared__ float sh_red[2][4][4];
    __shared__ f32x4 sh_part[2][4][2][32];
    const float bmul = (p.flags & GDN_FLAG_NEG_EIGVAL) ? 2.f : 1.f;

    for (int64_t t = 0; t < len; ++t) {
        const int pb = (int)(t & 1);
        const int64_t tok = bos + t;
        const float qv = to_f32(cur.q), kv = to_f32(cur.k);
        if constexpr (GK) {
            if (tid < 128) {
                float x = cur.gk;
                if (p.gk_act) {
                    x += gk_bias;
                    x = p.gk_act == 2 ? p.gk_lower * sigmoid_f(a_k * x) : -a_k * softplus_f(x);
                }
                const float e = __expf(x);
                sh_q[pb][tid] = qv * e; sh_k[pb][tid] = kv * e; sh_kr[pb][tid] = kv; sh_eg[pb][tid] = e;
            }
        } else {
            if (tid < 128) { sh_q[pb][tid] = qv; sh_k[pb][tid] = kv; }
        }
        float sqq = wave_sum(qv * qv), skk = wave_sum(kv * kv), sqk = wave_sum(qv * kv);
        if (lane == 0) { sh_red[pb][wave][0] = sqq; sh_red[pb][wave][1] = skk; sh_red[pb][wave][2] = sqk; }
        if constexpr (PK) {
            const float pv = to_f32(cur.pk);
            if (tid < 128) sh_p[pb][tid] = pv;
            const float spp = wave_sum(pv * pv);
            if (lane == 0) sh_red[pb][wave][3] = spp;
        }
        float eg = 1.f;
        if (p.g) {
            float gt = cur.g;
            if (p.A_log) gt = a_neg * softplus_f(gt + dtb);
            eg = __expf(gt);
        }
        float bb = cur.b;
        if (p.flags & GDN_FLAG_BETA_SIGMOID) bb = bmul * sigmoid_f(bb);
        const f32x4 vv = {to_f32(cur.v[0]), to_f32(cur.v[1]), to_f32(cur.v[2]), to_f32(cur.v[3])};
        if (t + 1 < len) cur = fetch(tok + 1);          // the next token's rows travel during this one's arithmetic
        __syncthreads();
        sqq = sh_red[pb][0][0] + sh_red[pb][1][0];      // (q and k live in waves 0 and 1)
        skk = sh_red[pb][0][1] + sh_red[pb][1][1];
        sqk = sh_red[pb][0][2] + sh_red[pb][1][2];
        float rq = p.scale, rk = 1.f, rp = 1.f;
        if (p.flags & GDN_FLAG_QK_L2NORM) {
            rq *= 1.f / sqrtf(sqq + 1e-6f);
            rk = 1.f / sqrtf(skk + 1e-6f);
            if constexpr (PK) rp = 1.f / sqrtf(sh_red[pb][0][3] + sh_red[pb][1][3] + 1e-6f);
        }
        const float qk = sqk * rq * rk;
        // S^T k and S^T q over this thread's rows (k, q unscaled: the row factors come after the reduction)
        f32x4 sk = {0.f, 0.f, 0.f, 0.f}, sq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            sk += S[i] * (PK ? sh_p[pb][r0 + 8 * i] : sh_k[pb][r0 + 8 * i]);
            sq += S[i] * sh_q[pb][r0 + 8 * i];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) { sk[j] += __shfl_xor(sk[j], 32, 64); sq[j] += __shfl_xor(sq[j], 32, 64); }
        if (lane < 32) { sh_part[pb][wave][0][c] = sk; sh_part[pb][wave][1][c] = sq; }
        __syncthreads();
        sk = (sh_part[pb][0][0][c] + sh_part[pb][1][0][c] + sh_part[pb][2][0][c] + sh_part[pb][3][0][c]) * (PK ? rp : eg * rk);
        sq = (sh_part[pb][0][1][c] + sh_part[pb][1][1][c] + sh_part[pb][2][1][c] + sh_part[pb][3][1][c]) * (eg * rq);
        const f32x4 d = bb * (vv - sk);
        const f32x4 dk = d * rk;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if constexpr (GK) S[i] = S[i] * (eg * sh_eg[pb][r0 + 8 * i]) + dk * sh_kr[pb][r0 + 8 * i];
            else S[i] = S[i] * eg + dk * sh_k[pb][r0 + 8 * i];
        }
        if (r0 == 0) {
            const f32x4 ov = sq + d * qk;
            T* po = o + (tok * HV + ihv) * 128 + 4 * c;
            po[0] = from_f32<T>(ov.x); po[1] = from_f32<T>(ov.y); po[2] = from_f32<T>(ov.z); po[3] = from_f32<T>(ov.w);
        }
    }
    if (p.ht) {
#pragma unroll
        for (int i = 0; i < 16; ++i) __builtin_nontemporal_store(S[i], (f32x4*)(p.ht + state_off + (r0 + 8 * i) * 128));
    }
}

// The common decode shape with V-first states [V][K] (the layout serving engines keep, `state_v_first`): thread
// (c = tid % 32, r0 = tid / 32) owns key features 4c .. 4c+3 of value rows r0 + 8i, so S^T k and S^T q are sums along a
// row: four products per thread and row, then over the 32 lanes that share the row.  The token's rows are requested
// before the state here as well (k and q as the thread's own four features, v through LDS), two workgroups share a CU.
// GK: a decay per key feature as well (the KDA operator): here a factor per column, the thread's own four.
template <typename T, bool GK = false>
__global__ __launch_bounds__(256, 2) void gdn_decode_vfirst_kernel(RecurrentParams p) {
    const int tid = threadIdx.x;
    const int c = tid & 31, r0 = tid >> 5;
    const int64_t inh = xcd_block(p);
    if (inh < 0) return;
    const int64_t in = inh / p.HV;
    const int ihv = (int)(inh % p.HV);
    const int H = p.H, HV = p.HV;
    const int ih = ihv / (HV / H);
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    int64_t bos, len;
    if (p.cu_seqlens) {
        bos = load_index(p.cu_seqlens, in, cu32);
        len = load_index(p.cu_seqlens, in + 1, cu32) - bos;
    } else {
        bos = in * p.T;
        len = p.T;
    }
    const int64_t slot = p.state_slots ? load_index(p.state_slots, in, p.flags & GDN_FLAG_SLOT_INT32) : in;
    const int64_t state_off = (slot * HV + ihv) * (int64_t)16384 + 4 * c;
    const T* q = (const T*)p.q; const T* k = (const T*)p.k; const T* v = (const T*)p.v; T* o = (T*)p.o;
    struct Token { T q[4], k[4]; T v; float g, b; f32x4 gk; };
    const float a_k = GK && p.gk_act ? (p.A_log ? __expf(p.A_log[ihv]) : (p.gk_act == 2 ? 1.f : __expf(1.f))) : 0.f;
    f32x4 gk_bias = {0.f, 0.f, 0.f, 0.f};
    if (GK && p.gk_act && p.gk_bias) gk_bias = *(const f32x4*)(p.gk_bias + ihv * 128 + 4 * c);
    auto fetch = [&](int64_t tok) {
        Token x;
        const T* pq = q + (tok * H + ih) * 128 + 4 * c;
        const T* pk = k + (tok * H + ih) * 128 + 4 * c;
#pragma unroll
        for (int j = 0; j < 4; ++j) { x.q[j] = pq[j]; x.k[j] = pk[j]; }
        x.gk = f32x4{0.f, 0.f, 0.f, 0.f};
        if constexpr (GK) x.gk = *(const f32x4*)(p.gk + (tok * HV + ihv) * 128 + 4 * c);
        x.v = from_f32<T>(0.f);
        if (tid < 128) x.v = v[(tok * HV + ihv) * 128 + tid];
        x.g = p.g ? load_scalar(p.g, tok * HV + ihv, p.gb_dtype) : 0.f;
        x.b = p.beta ? load_scalar(p.beta, tok * HV + ihv, p.gb_dtype) : 1.f;
        return x;
    };
    Token cur = {};
    if (len > 0) cur = fetch(bos);
    float a_neg = 0.f, dtb = 0.f;
    if (p.A_log) { a_neg = -__expf(p.A_log[ihv]); if (p.dt_bias) dtb = p.dt_bias[ihv]; }
    f32x4 S[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        S[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (p.h0) S[i] = __builtin_nontemporal_load((const f32x4*)(p.h0 + state_off + (r0 + 8 * i) * 128));
    }
    __shared__ float sh_v[2][128];
    const float bmul = (p.flags & GDN_FLAG_NEG_EIGVAL) ? 2.f : 1.f;
    auto row_sum = [&](float x) {                               // over the 32 lanes that share a row
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) x += __shfl_xor(x, off, 64);
        return x;
    };

    for (int64_t t = 0; t < len; ++t) {
        const int pb = (int)(t & 1);
        const int64_t tok = bos + t;
        f32x4 qc, kc;
#pragma unroll
        for (int j = 0; j < 4; ++j) { qc[j] = to_f32(cur.q[j]); kc[j] = to_f32(cur.k[j]); }
        if (tid < 128) sh_v[pb][tid] = to_f32(cur.v);
        float eg = 1.f;
        if (p.g) {
            float gt = cur.g;
            if (p.A_log) gt = a_neg * softplus_f(gt + dtb);
            eg = __expf(gt);
        }
        float bb = cur.b;
        if (p.flags & GDN_FLAG_BETA_SIGMOID) bb = bmul * sigmoid_f(bb);
        f32x4 eg4 = {eg, eg, eg, eg};
        if constexpr (GK) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float x = cur.gk[j];
                if (p.gk_act) {
                    x += gk_bias[j];
                    x = p.gk_act == 2 ? p.gk_lower * sigmoid_f(a_k * x) : -a_k * softplus_f(x);
                }
                eg4[j] *= __expf(x);
            }
        }
        if (t + 1 < len) cur = fetch(tok + 1);          // the next token's rows travel during this one's arithmetic
        const float sqq = row_sum(qc.x * qc.x + qc.y * qc.y + qc.z * qc.z + qc.w * qc.w);
        const float skk = row_sum(kc.x * kc.x + kc.y * kc.y + kc.z * kc.z + kc.w * kc.w);
        const float sqk = row_sum(qc.x * kc.x + qc.y * kc.y + qc.z * kc.z + qc.w * kc.w);
        float rq = p.scale, rk = 1.f;
        if (p.flags & GDN_FLAG_QK_L2NORM) {
            rq *= 1.f / sqrtf(sqq + 1e-6f);
            rk = 1.f / sqrtf(skk + 1e-6f);
        }
        const float qk = sqk * rq * rk;
        kc *= rk; qc *= rq;
        __syncthreads();                                // (v of this token is in LDS)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int row = r0 + 8 * i;
            const f32x4 sdec = S[i] * eg4;
            const f32x4 a = sdec * kc, b = sdec * qc;
            const float sk = row_sum((a.x + a.y) + (a.z + a.w)), sq = row_sum((b.x + b.y) + (b.z + b.w));
            const float d = bb * (sh_v[pb][row] - sk);
            S[i] = sdec + kc * d;
            if (c == 0) o[(tok * HV + ihv) * 128 + row] = from_f32<T>(sq + d * qk);
        }
    }
    if (p.ht) {
#pragma unroll
        for (int i = 0; i < 16; ++i) __builtin_nontemporal_store(S[i], (f32x4*)(p.ht + state_off + (r0 + 8 * i) * 128));
    }
}

// The same step with the states held in bf16 in memory (half the traffic of a decode step): K = V = 128, K-first.  The
// recurrence runs in fp32 registers; the state is rounded (to nearest even) once, when it is written back.  A thread owns
// 8 value columns (16 bytes of a row) of key rows r0 + 16 i; a wave instruction covers four whole rows.  (Three to five
// workgroups per CU run at the same speed, two are slower: no cap on the occupancy here.)
template <typename T>
__global__ __launch_bounds__(256, 2) void gdn_decode_bf16_kernel(RecurrentParams p) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = tid & 15, r0 = tid >> 4;
    const int64_t inh = xcd_block(p);
    if (inh < 0) return;
    const int64_t in = inh / p.HV;
    const int ihv = (int)(inh % p.HV);
    const int H = p.H, HV = p.HV;
    const int ih = ihv / (HV / H);
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    int64_t bos, len;
    if (p.cu_seqlens) {
        bos = load_index(p.cu_seqlens, in, cu32);
        len = load_index(p.cu_seqlens, in + 1, cu32) - bos;
    } else {
        bos = in * p.T;
        len = p.T;
    }
    const int64_t slot = p.state_slots ? load_index(p.state_slots, in, p.flags & GDN_FLAG_SLOT_INT32) : in;
    const int64_t state_off = (slot * HV + ihv) * (int64_t)16384 + 8 * c;
    const T* q = (const T*)p.q; const T* k = (const T*)p.k; const T* v = (const T*)p.v; T* o = (T*)p.o;
    struct Token { T q, k; T v[8]; float g, b; };
    auto fetch = [&](int64_t tok) {
        Token x;
        x.q = x.k = from_f32<T>(0.f);
        if (tid < 128) { x.q = q[(tok * H + ih) * 128 + tid]; x.k = k[(tok * H + ih) * 128 + tid]; }
        const T* pv = v + (tok * HV + ihv) * 128 + 8 * c;
#pragma unroll
        for (int j = 0; j < 8; ++j) x.v[j] = pv[j];
        x.g = p.g ? load_scalar(p.g, tok * HV + ihv, p.gb_dtype) : 0.f;
        x.b = p.beta ? load_scalar(p.beta, tok * HV + ihv, p.gb_dtype) : 1.f;
        return x;
    };
    Token cur = {};
    if (len > 0) cur = fetch(bos);
    float a_neg = 0.f, dtb = 0.f;
    if (p.A_log) { a_neg = -__expf(p.A_log[ihv]); if (p.dt_bias) dtb = p.dt_bias[ihv]; }
    // ---- the state: 8 requests of 16 bytes (8 bf16) per thread ----
    const bf16_t* h0 = (const bf16_t*)p.h0;
    u32x4 raw[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) raw[i] = __builtin_nontemporal_load((const u32x4*)(h0 + state_off + (r0 + 16 * i) * 128));
    __shared__ float sh_q[2][128], sh_k[2][128];
    __shared__ float sh_red[2][4][4];
    __shared__ float sh_part[2][4][2][128];
    const float bmul = (p.flags & GDN_FLAG_NEG_EIGVAL) ? 2.f : 1.f;
    float S[8][8];                                       // bf16 -> fp32: the 16 bits become the upper half of the word
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            S[i][2 * j] = __builtin_bit_cast(float, raw[i][j] << 16);
            S[i][2 * j + 1] = __builtin_bit_cast(float, raw[i][j] & 0xffff0000u);
        }

    for (int64_t t = 0; t < len; ++t) {
        const int pb = (int)(t & 1);
        const int64_t tok = bos + t;
        const float qv = to_f32(cur.q), kv = to_f32(cur.k);
        if (tid < 128) { sh_q[pb][tid] = qv; sh_k[pb][tid] = kv; }
        float sqq = wave_sum(qv * qv), skk = wave_sum(kv * kv), sqk = wave_sum(qv * kv);
        if (lane == 0) { sh_red[pb][wave][0] = sqq; sh_red[pb][wave][1] = skk; sh_red[pb][wave][2] = sqk; }
        float eg = 1.f;
        if (p.g) {
            float gt = cur.g;
            if (p.A_log) gt = a_neg * softplus_f(gt + dtb);
            eg = __expf(gt);
        }
        float bb = cur.b;
        if (p.flags & GDN_FLAG_BETA_SIGMOID) bb = bmul * sigmoid_f(bb);
        float vv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) vv[j] = to_f32(cur.v[j]);
        if (t + 1 < len) cur = fetch(tok + 1);
        __syncthreads();
        sqq = sh_red[pb][0][0] + sh_red[pb][1][0];
        skk = sh_red[pb][0][1] + sh_red[pb][1][1];
        sqk = sh_red[pb][0][2] + sh_red[pb][1][2];
        float rq = p.scale, rk = 1.f;
        if (p.flags & GDN_FLAG_QK_L2NORM) {
            rq *= 1.f / sqrtf(sqq + 1e-6f);
            rk = 1.f / sqrtf(skk + 1e-6f);
        }
        const float qk = sqk * rq * rk;
        float sk[8], sq[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) sk[j] = sq[j] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float kr = sh_k[pb][r0 + 16 * i], qr = sh_q[pb][r0 + 16 * i];
#pragma unroll
            for (int j = 0; j < 8; ++j) { sk[j] += S[i][j] * kr; sq[j] += S[i][j] * qr; }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            sk[j] += __shfl_xor(sk[j], 16, 64); sq[j] += __shfl_xor(sq[j], 16, 64);
            sk[j] += __shfl_xor(sk[j], 32, 64); sq[j] += __shfl_xor(sq[j], 32, 64);
        }
        if (lane < 16) {
#pragma unroll
            for (int j = 0; j < 8; ++j) { sh_part[pb][wave][0][8 * c + j] = sk[j]; sh_part[pb][wave][1][8 * c + j] = sq[j]; }
        }
        __syncthreads();
        float d[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int col = 8 * c + j;
            sk[j] = (sh_part[pb][0][0][col] + sh_part[pb][1][0][col] + sh_part[pb][2][0][col] + sh_part[pb][3][0][col]) * (eg * rk);
            sq[j] = (sh_part[pb][0][1][col] + sh_part[pb][1][1][col] + sh_part[pb][2][1][col] + sh_part[pb][3][1][col]) * (eg * rq);
            d[j] = bb * (vv[j] - sk[j]);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float kr = sh_k[pb][r0 + 16 * i] * rk;
#pragma unroll
            for (int j = 0; j < 8; ++j) S[i][j] = S[i][j] * eg + d[j] * kr;
        }
        if (r0 == 0) {
            T* po = o + (tok * HV + ihv) * 128 + 8 * c;
#pragma unroll
            for (int j = 0; j < 8; ++j) po[j] = from_f32<T>(sq[j] + d[j] * qk);
        }
    }
    if (p.ht) {
        bf16_t* ht = (bf16_t*)p.ht;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            u32x4 out;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bf16x2 pr = {(bf16_t)S[i][2 * j], (bf16_t)S[i][2 * j + 1]};
                out[j] = __builtin_bit_cast(uint32_t, pr);
            }
            __builtin_nontemporal_store(out, (u32x4*)(ht + state_off + (r0 + 16 * i) * 128));
        }
    }
}

// Grid for xcd_block(): launches that cover the chip several times over hand every XCD runs of `group` consecutive
// work items (the states of one sequence); smaller ones keep the plain order.
static int64_t place(RecurrentParams& p, int64_t nblocks, int64_t group) {
    p.nblocks = nblocks;
    p.xcd_group = 0;
    if (nblocks < 2048 || group >= (1 << 20)) return nblocks;
    p.xcd_group = (int)group;
    const int64_t ngroups = (nblocks + group - 1) / group;
    return (ngroups + 7) / 8 * 8 * group;
}

template <typename T, int KMAX, bool VFIRST>
static int launch_vb(const RecurrentParams& p0, int64_t n_states, int vb, hipStream_t stream) {
    RecurrentParams p = p0;
    p.NVB = (p.V + vb - 1) / vb;
    dim3 grid((unsigned)place(p, n_states * p.NVB, (int64_t)p.HV * p.NVB)), block(256);
    void (*kern)(RecurrentParams) = vb == 128 ? gdn_recurrent_kernel<T, KMAX, 128, VFIRST>
                                   : vb == 64 ? gdn_recurrent_kernel<T, KMAX, 64, VFIRST> : gdn_recurrent_kernel<T, KMAX, 32, VFIRST>;
    if constexpr (!VFIRST) {
        if (p.pk) kern = vb == 128 ? gdn_recurrent_kernel<T, KMAX, 128, false, true>
                       : vb == 64 ? gdn_recurrent_kernel<T, KMAX, 64, false, true> : gdn_recurrent_kernel<T, KMAX, 32, false, true>;
    }
    hipLaunchKernelGGL(kern, grid, block, 0, stream, p);
    return check_launch("gdn_recurrent_kernel");
}

template <typename T>
static int launch_t(const RecurrentParams& p, int64_t n_states, hipStream_t stream) {
    const bool vfirst = p.flags & GDN_FLAG_STATE_V_FIRST;
    if (p.flags & GDN_FLAG_STATE_BF16) {
        RecurrentParams pd = p;
        const int64_t grid = place(pd, n_states, p.HV);
        hipLaunchKernelGGL(gdn_decode_bf16_kernel<T>, dim3((unsigned)grid), dim3(256), 0, stream, pd);
        return check_launch("gdn_decode_bf16_kernel");
    }
    if (p.K == 128 && p.V == 128 && vfirst && !p.gv && !p.pk && n_states >= 1024 && (uintptr_t)p.gk_bias % 16 == 0 &&
        !(p.flags & (GDN_FLAG_BETA_VECTOR | GDN_FLAG_SLOT_PER_TOKEN | GDN_FLAG_STATE_PER_TOKEN))) {
        RecurrentParams pd = p;
        const int64_t grid = place(pd, n_states, p.HV);
        static SmemAttrDone attr_done_vf, attr_done_vf_gk;
        if (p.gk) {
            if (int rc = ensure_dynamic_smem((const void*)gdn_decode_vfirst_kernel<T, true>, DECODE_LDS_PAD, attr_done_vf_gk, "hipFuncSetAttribute(decode)")) return rc;
            hipLaunchKernelGGL((gdn_decode_vfirst_kernel<T, true>), dim3((unsigned)grid), dim3(256), DECODE_LDS_PAD, stream, pd);
        } else {
            if (int rc = ensure_dynamic_smem((const void*)gdn_decode_vfirst_kernel<T, false>, DECODE_LDS_PAD, attr_done_vf, "hipFuncSetAttribute(decode)")) return rc;
            hipLaunchKernelGGL((gdn_decode_vfirst_kernel<T, false>), dim3((unsigned)grid), dim3(256), DECODE_LDS_PAD, stream, pd);
        }
        return check_launch("gdn_decode_vfirst_kernel");
    }
    // the common decode shape has a kernel of its own (enough states to fill the chip with whole-state workgroups)
    if (p.K == 128 && p.V == 128 && !vfirst && !p.gv && !(p.pk && p.gk) && n_states >= 1024 &&
        !(p.flags & (GDN_FLAG_BETA_VECTOR | GDN_FLAG_SLOT_PER_TOKEN | GDN_FLAG_STATE_PER_TOKEN))) {
        RecurrentParams pd = p;
        const int64_t grid = place(pd, n_states, p.HV);
        static SmemAttrDone attr_done, attr_done_gk, attr_done_pk;     // per instantiation
        if (p.pk) {
            if (int rc = ensure_dynamic_smem((const void*)gdn_decode_kernel<T, false, true>, DECODE_LDS_PAD, attr_done_pk, "hipFuncSetAttribute(decode)")) return rc;
            hipLaunchKernelGGL((gdn_decode_kernel<T, false, true>), dim3((unsigned)grid), dim3(256), DECODE_LDS_PAD, stream, pd);
        } else if (p.gk) {
            if (int rc = ensure_dynamic_smem((const void*)gdn_decode_kernel<T, true>, DECODE_LDS_PAD, attr_done_gk, "hipFuncSetAttribute(decode)")) return rc;
            hipLaunchKernelGGL((gdn_decode_kernel<T, true>), dim3((unsigned)grid), dim3(256), DECODE_LDS_PAD, stream, pd);
        } else {
            if (int rc = ensure_dynamic_smem((const void*)gdn_decode_kernel<T, false>, DECODE_LDS_PAD, attr_done, "hipFuncSetAttribute(decode)")) return rc;
            hipLaunchKernelGGL((gdn_decode_kernel<T, false>), dim3((unsigned)grid), dim3(256), DECODE_LDS_PAD, stream, pd);
        }
        return check_launch("gdn_decode_kernel");
    }
    // Value block per workgroup: whole rows when there are enough (sequence, head) pairs to
    // fill 256 CUs several times over, narrower blocks otherwise.
    int vb = 128;
    while (vb > 32 && (p.V <= vb / 2 || n_states * ((p.V + vb - 1) / vb) < 1024)) vb >>= 1;
    if (vfirst) vb = p.V >= 64 && n_states >= 1024 ? 64 : 32;   // V-first rows are independent; keep R small
    const int kmax = p.K <= 64 ? 64 : (p.K <= 128 ? 128 : 256);
#define GDN_REC_CASE(KM)                                                          \
    case KM:                                                                      \
        return vfirst ? launch_vb<T, KM, true>(p, n_states, vb, stream)           \
                      : launch_vb<T, KM, false>(p, n_states, vb, stream);
    switch (kmax) {
        GDN_REC_CASE(64)
        GDN_REC_CASE(128)
        GDN_REC_CASE(256)
    }
#undef GDN_REC_CASE
    return GDN_ERR_UNSUPPORTED;
}

}  // namespace gdn

// gk_act, gk_bias, gk_lower: see RecurrentParams (0, NULL, 0 for the gated delta rule)
static int recurrent_entry(
    const char* who,
    const void* q, const void* k, const void* v,
    const void* g, const void* beta, const float* gk, const float* gv,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* state_slots, const void* num_accepted, int64_t slots_stride,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V, int64_t N,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream,
    int gk_act, const float* gk_bias, float gk_lower, const void* pk = nullptr) {
    using namespace gdn;
    GDN_CHECK_ARG(T == 0 || (q && k && v && o), GDN_ERR_INVALID, "%s: q, k, v, o must not be NULL", who);
    GDN_CHECK_ARG(B >= 1 && T >= 0 && H >= 1 && HV >= 1 && K >= 1 && V >= 1 && N >= 1, GDN_ERR_INVALID,
                  "%s: non-positive dimension", who);
    GDN_CHECK_ARG(HV % H == 0, GDN_ERR_INVALID, "%s: HV=%lld not divisible by H=%lld", who,
                  (long long)HV, (long long)H);
    GDN_CHECK_ARG(cu_seqlens ? B == 1 : N == B, GDN_ERR_INVALID,
                  "%s: with cu_seqlens B must be 1; without it N must equal B", who);
    GDN_CHECK_ARG(K <= 256, GDN_ERR_UNSUPPORTED, "%s: K=%lld > 256", who, (long long)K);
    GDN_CHECK_ARG(K % 4 == 0 && V % 4 == 0, GDN_ERR_UNSUPPORTED,
                  "%s: K=%lld and V=%lld must be multiples of 4", who, (long long)K, (long long)V);
    GDN_CHECK_ARG((N + 8) * HV * ((V + 31) / 32) < (1ll << 31), GDN_ERR_UNSUPPORTED, "%s: grid too large", who);
    GDN_CHECK_ARG(((uintptr_t)h0 % 16) == 0 && ((uintptr_t)ht % 16) == 0 && ((uintptr_t)gk % 16) == 0 &&
                      ((uintptr_t)gv % 16) == 0,
                  GDN_ERR_INVALID, "%s: h0/ht/gk/gv must be 16-byte aligned", who);
    GDN_CHECK_ARG(!(A_log && !g && !gk_act), GDN_ERR_INVALID, "%s: A_log given without g", who);
    GDN_CHECK_ARG(!(flags & GDN_FLAG_SLOT_PER_TOKEN) || (state_slots && h0 && slots_stride >= 1), GDN_ERR_INVALID,
                  "%s: GDN_FLAG_SLOT_PER_TOKEN needs state_slots, the pool as h0 and slots_stride >= 1", who);
    GDN_CHECK_ARG(!num_accepted || (flags & GDN_FLAG_SLOT_PER_TOKEN), GDN_ERR_INVALID,
                  "%s: num_accepted needs GDN_FLAG_SLOT_PER_TOKEN", who);
    GDN_CHECK_ARG(!((flags & GDN_FLAG_SLOT_PER_TOKEN) && (flags & GDN_FLAG_STATE_PER_TOKEN)), GDN_ERR_INVALID,
                  "%s: GDN_FLAG_SLOT_PER_TOKEN and GDN_FLAG_STATE_PER_TOKEN exclude each other", who);
    GDN_CHECK_ARG(!(flags & GDN_FLAG_STATE_BF16) ||
                      (h0 && K == 128 && V == 128 && !gk && !gv &&
                       !(flags & (GDN_FLAG_STATE_V_FIRST | GDN_FLAG_BETA_VECTOR | GDN_FLAG_SLOT_PER_TOKEN | GDN_FLAG_STATE_PER_TOKEN))),
                  GDN_ERR_UNSUPPORTED,
                  "%s: bf16 states need h0, K = V = 128, the K-first layout, no gk / gv / beta per column and states per sequence or slot", who);
    GDN_CHECK_ARG(!(flags & GDN_FLAG_STATE_PER_TOKEN) || (ht && ht != h0), GDN_ERR_INVALID,
                  "%s: GDN_FLAG_STATE_PER_TOKEN needs ht [tokens,HV,K,V] distinct from h0", who);
    hipStream_t s = (hipStream_t)stream;
    if (T == 0) {
        // no token: the final states are the initial ones (nothing to do for pools and per-token states)
        if (ht && !state_slots && !(flags & GDN_FLAG_STATE_PER_TOKEN)) return launch_state_copy(h0, ht, N * HV * K * V / ((flags & GDN_FLAG_STATE_BF16) ? 2 : 1), s);
        return GDN_OK;
    }
    RecurrentParams p;
    p.q = q; p.k = k; p.v = v; p.pk = pk; p.g = g; p.beta = beta; p.gk = gk; p.gv = gv;
    p.A_log = A_log; p.dt_bias = dt_bias; p.h0 = h0; p.ht = ht; p.o = o; p.cu_seqlens = cu_seqlens; p.state_slots = state_slots;
    p.num_accepted = num_accepted; p.slots_stride = slots_stride;
    p.T = T; p.H = (int)H; p.HV = (int)HV; p.K = (int)K; p.V = (int)V; p.NVB = 1;
    p.scale = scale; p.gb_dtype = gb_dtype; p.flags = flags;
    p.gk_act = gk_act; p.gk_bias = gk_bias; p.gk_lower = gk_lower;
    switch (qkv_dtype) {
        case GDN_DTYPE_BF16: return launch_t<bf16_t>(p, N * HV, s);
        case GDN_DTYPE_F16: return launch_t<f16_t>(p, N * HV, s);
        case GDN_DTYPE_F32: return launch_t<float>(p, N * HV, s);
    }
    set_error("%s: unknown qkv_dtype %d", who, qkv_dtype);
    return GDN_ERR_INVALID;
}

extern "C" int gdn_fused_recurrent_fwd(
    const void* q, const void* k, const void* v,
    const void* g, const void* beta, const float* gk, const float* gv,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* state_slots, const void* num_accepted, int64_t slots_stride,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V, int64_t N,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    return recurrent_entry("gdn_fused_recurrent_fwd", q, k, v, g, beta, gk, gv, A_log, dt_bias, h0, ht, o, cu_seqlens, state_slots,
                           num_accepted, slots_stride, B, T, H, HV, K, V, N, scale, qkv_dtype, gb_dtype, flags, stream, 0, nullptr, 0.f);
}

// The KDA operator's token recurrence: the gated delta rule with a decay per key feature, g [B,T,HV,K].
extern "C" int gdn_fused_recurrent_kda_fwd(
    const void* q, const void* k, const void* v,
    const float* g, const void* beta,
    const float* A_log, const float* dt_bias, float lower_bound, int gate_mode,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* state_slots, const void* num_accepted, int64_t slots_stride,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V, int64_t N,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    const char* who = "gdn_fused_recurrent_kda_fwd";
    GDN_CHECK_ARG(T == 0 || g, GDN_ERR_INVALID, "%s: g must not be NULL", who);
    GDN_CHECK_ARG(gate_mode >= 0 && gate_mode <= 2, GDN_ERR_INVALID, "%s: gate_mode %d is not 0 (log decays), 1 (softplus) or 2 (bounded sigmoid)", who, gate_mode);
    GDN_CHECK_ARG(gate_mode != 0 || (!A_log && !dt_bias), GDN_ERR_INVALID, "%s: A_log and dt_bias belong to the gate activation (gate_mode 1 or 2)", who);
    GDN_CHECK_ARG(!(flags & GDN_FLAG_STATE_BF16), GDN_ERR_UNSUPPORTED, "%s: bf16 states are not supported with a decay per key feature", who);
    return recurrent_entry(who, q, k, v, nullptr, beta, g, nullptr, A_log, nullptr, h0, ht, o, cu_seqlens, state_slots,
                           num_accepted, slots_stride, B, T, H, HV, K, V, N, scale, qkv_dtype, gb_dtype, flags, stream, gate_mode, dt_bias, lower_bound);
}

// The comba operator's token recurrence: a second key p [B,T,H,K] for the prediction, made before the token's decay.
extern "C" int gdn_fused_recurrent_comba_fwd(
    const void* q, const void* k, const void* p, const void* v,
    const void* g, const void* beta,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V, int64_t N,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    const char* who = "gdn_fused_recurrent_comba_fwd";
    GDN_CHECK_ARG(T == 0 || (p && g), GDN_ERR_INVALID, "%s: p and g must not be NULL", who);
    GDN_CHECK_ARG((flags & ~(uint32_t)(GDN_FLAG_CU_INT32 | GDN_FLAG_QK_L2NORM | GDN_FLAG_BETA_VECTOR)) == 0, GDN_ERR_UNSUPPORTED,
                  "%s: only GDN_FLAG_CU_INT32, GDN_FLAG_QK_L2NORM (q, k and p) and GDN_FLAG_BETA_VECTOR are understood here", who);
    return recurrent_entry(who, q, k, v, g, beta, nullptr, nullptr, nullptr, nullptr, h0, ht, o, cu_seqlens, nullptr, nullptr, 0,
                           B, T, H, HV, K, V, N, scale, qkv_dtype, gb_dtype, flags, stream, 0, nullptr, 0.f, p);
}
