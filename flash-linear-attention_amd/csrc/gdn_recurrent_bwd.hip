// Backward of the token recurrence of the delta rule without gates (fused_recurrent_delta_rule) for gfx950.
//
//   forward, per (sequence, head):   u_t = v_t - S^T k_t;   S <- S + k_t (beta_t u_t)^T;   o_t = scale S^T q_t
//
// One WAVE owns the state of one (sequence, head) restricted to a block of VB value columns, [K][VB] fp32 in
// registers (64 per lane: lane (rg, cg) holds RPL key rows x CPL value columns), and walks the sequence three times:
//   pass A  forwards:  u_t (the residual the backward needs; kept in a workspace, not by the forward operator)
//   pass B  backwards: dS += scale q_t do_t^T;  dk_t = dS (beta_t u_t);  dvr = dS^T k_t;  dbeta_t = <dvr, u_t>;
//                      dv_t = beta_t dvr;  dS -= k_t dv_t^T;  at the start of the sequence dS is the gradient of h0
//   pass C  forwards:  dk_t -= S_{t-1} dv_t  (v_t's dependence on the state);  S <- S + k_t (beta_t u_t)^T;  dq_t = scale S do_t
// (the two-pass structure of fla/ops/delta_rule/fused_recurrent.py:111-266, which keeps u from its forward kernel).
// Sums over value columns stay inside the 4 lanes of a row group, sums over key rows run across the 16 row groups:
// cross-lane adds, no LDS, no barrier.  dq, dk (and dbeta per head) are partial over the value blocks; the host adds them.
#include "gdn_common.h"

namespace gdn {

struct RecurrentBwdParams {
    const void* q; const void* k; const void* v; const void* beta; const void* dout;
    const float* h0; const float* dht;
    float* dq_part; float* dk_part;      // [NVB][tokens][H][K]
    float* dv;                           // [tokens][H][V]
    float* db;                           // scalar beta: [NVB][tokens][H]; beta per column: [tokens][H][V]
    float* dh0;                          // [N][H][K][V] or NULL
    float* u;                            // workspace [tokens][H][V]
    const void* cu_seqlens;
    int64_t T, tokens;
    int H, K, V, NVB;
    float scale; int gb_dtype; uint32_t flags;
};

template <typename T, int N>
__device__ __forceinline__ void load_row(const T* p, bool ok, float (&x)[N]) {
    if constexpr (sizeof(T) == 2) {
        constexpr int W = N % 8 == 0 ? 8 : 4;               // 16- or 8-byte pieces
        typedef T VW __attribute__((ext_vector_type(W)));
#pragma unroll
        for (int i = 0; i < N; i += W) {
            VW t;
            if (ok) t = *(const VW*)(p + i);
#pragma unroll
            for (int e = 0; e < W; ++e) x[i + e] = ok ? (float)t[e] : 0.f;
        }
    } else {
#pragma unroll
        for (int i = 0; i < N; i += 4) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (ok) t = *(const f32x4*)(p + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) x[i + e] = t[e];
        }
    }
}
template <int N>
__device__ __forceinline__ void load_row_f32(const float* p, float (&x)[N]) {
#pragma unroll
    for (int i = 0; i < N; i += 4) {
        const f32x4 t = *(const f32x4*)(p + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[i + e] = t[e];
    }
}
template <int N>
__device__ __forceinline__ void store_row_f32(float* p, const float (&x)[N]) {
#pragma unroll
    for (int i = 0; i < N; i += 4) *(f32x4*)(p + i) = f32x4{x[i], x[i + 1], x[i + 2], x[i + 3]};
}

// KMAX = 128: 32 value columns per wave (8 rows x 8 columns per lane); KMAX = 256: 16 columns (16 rows x 4 columns).
// K is a multiple of 16 (<= KMAX), V a multiple of the block: the host pads.
template <typename T, int KMAX>
__global__ __launch_bounds__(64) void gdn_recurrent_delta_bwd_kernel(RecurrentBwdParams p) {
    constexpr int RPL = KMAX / 16, VB = KMAX == 128 ? 32 : 16, CPL = VB / 4;
    const int lane = threadIdx.x, cg = lane & 3, rg = lane >> 2;
    const int ivb = (int)(blockIdx.x % p.NVB);
    const int64_t inh = blockIdx.x / p.NVB;
    const int64_t n = inh / p.H;
    const int h = (int)(inh % p.H);
    const int K = p.K, V = p.V, H = p.H;
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32, beta_vec = p.flags & GDN_FLAG_BETA_VECTOR;
    int64_t bos, len;
    if (p.cu_seqlens) {
        bos = load_index(p.cu_seqlens, n, cu32);
        len = load_index(p.cu_seqlens, n + 1, cu32) - bos;
    } else {
        bos = n * p.T;
        len = p.T;
    }
    const int r0 = rg * RPL, c0 = ivb * VB + cg * CPL;
    const bool row_ok = r0 < K;                               // (K is a multiple of 16 = the rows of two lanes at KMAX = 128)
    const T* qg = (const T*)p.q;
    const T* kg = (const T*)p.k;
    const T* vg = (const T*)p.v;
    const T* dog = (const T*)p.dout;

    auto sum_cols = [&](float x) {                          // over the 4 lanes of a row group
        x += __shfl_xor(x, 1, 64);
        x += __shfl_xor(x, 2, 64);
        return x;
    };
    auto sum_rows = [&](float x) {                          // over the 16 row groups
#pragma unroll
        for (int o = 4; o < 64; o <<= 1) x += __shfl_xor(x, o, 64);
        return x;
    };
    auto beta_of = [&](int64_t tok, float (&b)[CPL]) {
        if (beta_vec) {
#pragma unroll
            for (int j = 0; j < CPL; ++j) b[j] = load_scalar(p.beta, (tok * H + h) * V + c0 + j, p.gb_dtype);
        } else {
            const float s = p.beta ? load_scalar(p.beta, tok * H + h, p.gb_dtype) : 1.f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) b[j] = s;
        }
    };
    auto state_off = [&](int i) { return inh * (int64_t)K * V + (int64_t)(r0 + i) * V + c0; };

    float S[RPL][CPL];
    auto load_state = [&](const float* src) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            float row[CPL];
            if (src && row_ok) load_row_f32<CPL>(src + state_off(i), row);
#pragma unroll
            for (int j = 0; j < CPL; ++j) S[i][j] = (src && row_ok) ? row[j] : 0.f;
        }
    };

    // ---- pass A: u_t = v_t - S^T k_t ----
    load_state(p.h0);
    for (int64_t t = 0; t < len; ++t) {
        const int64_t tok = bos + t;
        float kk[RPL], vv[CPL], bb[CPL];
        load_row<T, RPL>(kg + (tok * H + h) * K + r0, row_ok, kk);
        load_row<T, CPL>(vg + (tok * H + h) * V + c0, true, vv);
        beta_of(tok, bb);
        float u[CPL];
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < RPL; ++i) s += S[i][j] * kk[i];
            u[j] = vv[j] - sum_rows(s);
        }
        if (rg == 0) store_row_f32<CPL>(p.u + (tok * H + h) * V + c0, u);
#pragma unroll
        for (int i = 0; i < RPL; ++i)
#pragma unroll
            for (int j = 0; j < CPL; ++j) S[i][j] += kk[i] * (bb[j] * u[j]);
    }
    __threadfence();                                          // u is read again below by other lanes of this wave

    // ---- pass B, backwards: S holds dS ----
    load_state(p.dht);
    for (int64_t t = len - 1; t >= 0; --t) {
        const int64_t tok = bos + t;
        float kk[RPL], qq[RPL], dd[CPL], u[CPL], bb[CPL];
        load_row<T, RPL>(kg + (tok * H + h) * K + r0, row_ok, kk);
        load_row<T, RPL>(qg + (tok * H + h) * K + r0, row_ok, qq);
        load_row<T, CPL>(dog + (tok * H + h) * V + c0, true, dd);
        load_row_f32<CPL>(p.u + (tok * H + h) * V + c0, u);
        beta_of(tok, bb);
#pragma unroll
        for (int i = 0; i < RPL; ++i)
#pragma unroll
            for (int j = 0; j < CPL; ++j) S[i][j] += p.scale * qq[i] * dd[j];
        float dk[RPL];
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) s += S[i][j] * (bb[j] * u[j]);
            dk[i] = sum_cols(s);
        }
        if (cg == 0 && row_ok) store_row_f32<RPL>(p.dk_part + ((ivb * p.tokens + tok) * H + h) * K + r0, dk);
        float dv[CPL], dbv[CPL], dbs = 0.f;
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < RPL; ++i) s += S[i][j] * kk[i];
            s = sum_rows(s);
            dbv[j] = s * u[j];
            dbs += dbv[j];
            dv[j] = s * bb[j];
        }
        if (rg == 0) {
            store_row_f32<CPL>(p.dv + (tok * H + h) * V + c0, dv);
            if (beta_vec) store_row_f32<CPL>(p.db + (tok * H + h) * V + c0, dbv);
        }
        if (!beta_vec) {
            dbs = sum_cols(dbs);
            if (lane == 0) p.db[(ivb * p.tokens + tok) * H + h] = dbs;
        }
#pragma unroll
        for (int i = 0; i < RPL; ++i)
#pragma unroll
            for (int j = 0; j < CPL; ++j) S[i][j] -= kk[i] * dv[j];
    }
    if (p.dh0 && row_ok) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) store_row_f32<CPL>(p.dh0 + state_off(i), S[i]);
    }
    __threadfence();                                          // dv and the first part of dk are read again below

    // ---- pass C, forwards: S is the state again ----
    load_state(p.h0);
    for (int64_t t = 0; t < len; ++t) {
        const int64_t tok = bos + t;
        float kk[RPL], dd[CPL], u[CPL], dv[CPL], bb[CPL], dk[RPL];
        load_row<T, RPL>(kg + (tok * H + h) * K + r0, row_ok, kk);
        load_row<T, CPL>(dog + (tok * H + h) * V + c0, true, dd);
        load_row_f32<CPL>(p.u + (tok * H + h) * V + c0, u);
        load_row_f32<CPL>(p.dv + (tok * H + h) * V + c0, dv);
        beta_of(tok, bb);
        float* dkp = p.dk_part + ((ivb * p.tokens + tok) * H + h) * K + r0;
        if (cg == 0 && row_ok) load_row_f32<RPL>(dkp, dk);
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) s += S[i][j] * dv[j];
            s = sum_cols(s);
            if (cg == 0 && row_ok) dk[i] -= s;
        }
        if (cg == 0 && row_ok) store_row_f32<RPL>(dkp, dk);
#pragma unroll
        for (int i = 0; i < RPL; ++i)
#pragma unroll
            for (int j = 0; j < CPL; ++j) S[i][j] += kk[i] * (bb[j] * u[j]);
        float dq[RPL];
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) s += S[i][j] * dd[j];
            dq[i] = p.scale * sum_cols(s);
        }
        if (cg == 0 && row_ok) store_row_f32<RPL>(p.dq_part + ((ivb * p.tokens + tok) * H + h) * K + r0, dq);
    }
}

template <typename T>
static int launch_recurrent_delta_bwd(const RecurrentBwdParams& p, int64_t N, hipStream_t s) {
    const int64_t blocks = N * p.H * p.NVB;
    if (blocks <= 0) return GDN_OK;
    if (p.K <= 128) hipLaunchKernelGGL((gdn_recurrent_delta_bwd_kernel<T, 128>), dim3((unsigned)blocks), dim3(64), 0, s, p);
    else hipLaunchKernelGGL((gdn_recurrent_delta_bwd_kernel<T, 256>), dim3((unsigned)blocks), dim3(64), 0, s, p);
    return check_launch("gdn_recurrent_delta_bwd_kernel");
}

}  // namespace gdn

extern "C" int64_t gdn_fused_recurrent_delta_bwd_value_block(int64_t K) { return K <= 128 ? 32 : 16; }

extern "C" int gdn_fused_recurrent_delta_bwd(
    const void* q, const void* k, const void* v, const void* beta, const void* dout, const float* h0, const float* dht,
    float* dq_part, float* dk_part, float* dv, float* db, float* dh0, float* u_workspace, const void* cu_seqlens,
    int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N, float scale, int qkv_dtype, int gb_dtype, uint32_t flags,
    void* stream) {
    using namespace gdn;
    const char* who = "gdn_fused_recurrent_delta_bwd";
    GDN_CHECK_ARG(B >= 1 && T >= 0 && H >= 1 && N >= 1, GDN_ERR_INVALID, "%s: non-positive dimension", who);
    GDN_CHECK_ARG(K >= 16 && K % 16 == 0 && K <= 256, GDN_ERR_UNSUPPORTED, "%s: K must be a multiple of 16 up to 256 (got %lld)", who, (long long)K);
    const int64_t VB = gdn_fused_recurrent_delta_bwd_value_block(K);
    GDN_CHECK_ARG(V >= VB && V % VB == 0, GDN_ERR_UNSUPPORTED, "%s: V must be a multiple of %lld (got %lld)", who, (long long)VB, (long long)V);
    GDN_CHECK_ARG(qkv_dtype == GDN_DTYPE_BF16 || qkv_dtype == GDN_DTYPE_F16 || qkv_dtype == GDN_DTYPE_F32, GDN_ERR_UNSUPPORTED, "%s: bad dtype", who);
    GDN_CHECK_ARG(!(flags & ~(uint32_t)(GDN_FLAG_CU_INT32 | GDN_FLAG_BETA_VECTOR)), GDN_ERR_UNSUPPORTED, "%s: unsupported flag", who);
    GDN_CHECK_ARG(!(flags & GDN_FLAG_BETA_VECTOR) || beta, GDN_ERR_INVALID, "%s: GDN_FLAG_BETA_VECTOR without beta", who);
    if (cu_seqlens) GDN_CHECK_ARG(B == 1, GDN_ERR_INVALID, "%s: with cu_seqlens B must be 1", who);
    else GDN_CHECK_ARG(N == B, GDN_ERR_INVALID, "%s: without cu_seqlens N must equal B", who);
    if (T == 0) return GDN_OK;
    GDN_CHECK_ARG(q && k && v && dout && dq_part && dk_part && dv && db && u_workspace, GDN_ERR_INVALID, "%s: NULL tensor", who);
    GDN_CHECK_ARG(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)dout | (uintptr_t)h0 | (uintptr_t)dht | (uintptr_t)dq_part |
                   (uintptr_t)dk_part | (uintptr_t)dv | (uintptr_t)db | (uintptr_t)dh0 | (uintptr_t)u_workspace) % 16 == 0,
                  GDN_ERR_INVALID, "%s: tensors must be 16-byte aligned", who);
    RecurrentBwdParams p;
    p.q = q; p.k = k; p.v = v; p.beta = beta; p.dout = dout; p.h0 = h0; p.dht = dht;
    p.dq_part = dq_part; p.dk_part = dk_part; p.dv = dv; p.db = db; p.dh0 = dh0; p.u = u_workspace; p.cu_seqlens = cu_seqlens;
    p.T = T; p.tokens = B * T; p.H = (int)H; p.K = (int)K; p.V = (int)V; p.NVB = (int)(V / VB);
    p.scale = scale; p.gb_dtype = gb_dtype; p.flags = flags;
    hipStream_t s = (hipStream_t)stream;
    if (qkv_dtype == GDN_DTYPE_BF16) return launch_recurrent_delta_bwd<bf16_t>(p, N, s);
    if (qkv_dtype == GDN_DTYPE_F16) return launch_recurrent_delta_bwd<f16_t>(p, N, s);
    return launch_recurrent_delta_bwd<float>(p, N, s);
}
