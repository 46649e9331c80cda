// Row-wise l2 normalisation of q and k around the backward pass of the chunked operator, and the last step of that
// pass for dq and dk (sum over the value heads of a q/k head, then back through the normalisation).  Streaming kernels:
// a group of lanes per row, 16 bytes per lane.
#include "gdn_common.h"

namespace gdn {

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> { typedef bf16x8 type; };
template <> struct Vec8<f16_t> { typedef f16x8 type; };

template <int L>
__device__ __forceinline__ float sum_over_group(float x) {       // over L consecutive lanes (L a power of two)
#pragma unroll
    for (int off = 1; off < L; off <<= 1) x += __shfl_xor(x, off, 64);
    return x;
}

// y[row][0..Dout) = x[row][0..D) / sqrt(sum x^2 + 1e-6), zeros from D on; rstd[row] = the factor
template <typename T, int L>
__global__ __launch_bounds__(256) void gdn_l2norm_fwd_kernel(const T* x, T* y, float* rstd, int64_t rows, int D, int Dout) {
    typedef typename Vec8<T>::type V8;
    const int sub = threadIdx.x % L;
    const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / L;
    if (row >= rows) return;                                     // (whole groups leave together)
    V8 v;
    float f[8], ss = 0.f;
    const bool in = sub * 8 < D;
    if (in) v = *(const V8*)(x + row * D + sub * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) { f[e] = in ? (float)v[e] : 0.f; ss += f[e] * f[e]; }
    const float r = rsqrtf(sum_over_group<L>(ss) + 1e-6f);
    if (sub * 8 < Dout) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (T)(f[e] * r);
        *(V8*)(y + row * Dout + sub * 8) = v;
    }
    if (sub == 0) rstd[row] = r;
}

// dx[row][0..Dout) = back through the normalisation of  sum_g dxh[row][g][0..Din):
// with y (normalised rows, Din wide) and rstd:  (dy - y <dy, y>) rstd;  without: dy
template <typename T, int L>
__global__ __launch_bounds__(256) void gdn_l2norm_bwd_kernel(const T* dxh, const T* y, const float* rstd, T* dx, int64_t rows,
                                                             int G, int Din, int Dout) {
    typedef typename Vec8<T>::type V8;
    const int sub = threadIdx.x % L;
    const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / L;
    if (row >= rows) return;
    float dy[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const bool in = sub * 8 < Din;
    if (in) {
        for (int g = 0; g < G; ++g) {
            const V8 v = *(const V8*)(dxh + (row * G + g) * Din + sub * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) dy[e] += (float)v[e];
        }
    }
    if (y) {
        V8 yv;
        float dot = 0.f, yf[8];
        if (in) yv = *(const V8*)(y + row * Din + sub * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) { yf[e] = in ? (float)yv[e] : 0.f; dot += dy[e] * yf[e]; }
        dot = sum_over_group<L>(dot);
        const float r = rstd[row];
#pragma unroll
        for (int e = 0; e < 8; ++e) dy[e] = (dy[e] - yf[e] * dot) * r;
    }
    if (sub * 8 < Dout) {
        V8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (T)dy[e];
        *(V8*)(dx + row * Dout + sub * 8) = o;
    }
}

template <typename T>
static int launch_l2norm(const void* x, void* y, float* rstd, const void* dxh, int64_t rows, int G, int D, int Dout, bool bwd,
                         hipStream_t s) {
    const int wide = D > Dout ? D : Dout;
    const int L = wide <= 64 ? 8 : wide <= 128 ? 16 : 32;
    const unsigned grid = (unsigned)((rows * L + 255) / 256);
#define GDN_L2_CASE(LL)                                                                                                             \
    case LL:                                                                                                                        \
        if (bwd) hipLaunchKernelGGL((gdn_l2norm_bwd_kernel<T, LL>), dim3(grid), dim3(256), 0, s, (const T*)dxh, (const T*)x, rstd,   \
                                    (T*)y, rows, G, D, Dout);                                                                       \
        else hipLaunchKernelGGL((gdn_l2norm_fwd_kernel<T, LL>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)y, rstd, rows, D, Dout); \
        break;
    switch (L) {
        GDN_L2_CASE(8)
        GDN_L2_CASE(16)
        GDN_L2_CASE(32)
    }
#undef GDN_L2_CASE
    return check_launch(bwd ? "gdn_l2norm_bwd_kernel" : "gdn_l2norm_fwd_kernel");
}

static int l2_args_ok(const char* who, int64_t rows, int64_t D, int64_t Dout, int dtype) {
    GDN_CHECK_ARG(rows >= 0 && rows * 32 < (1ll << 39), GDN_ERR_INVALID, "%s: bad number of rows", who);
    GDN_CHECK_ARG(D >= 8 && D % 8 == 0 && D <= 256 && Dout >= 8 && Dout % 8 == 0 && Dout <= 256, GDN_ERR_UNSUPPORTED,
                  "%s: row lengths must be multiples of 8 up to 256 (got %lld, %lld)", who, (long long)D, (long long)Dout);
    GDN_CHECK_ARG(dtype == GDN_DTYPE_BF16 || dtype == GDN_DTYPE_F16, GDN_ERR_UNSUPPORTED, "%s: bf16 or f16 only", who);
    return GDN_OK;
}

}  // namespace gdn

extern "C" int gdn_l2norm_fwd(const void* x, void* y, float* rstd, int64_t rows, int64_t D, int64_t Dout, int dtype, void* stream) {
    using namespace gdn;
    const char* who = "gdn_l2norm_fwd";
    if (int rc = l2_args_ok(who, rows, D, Dout, dtype)) return rc;
    GDN_CHECK_ARG(Dout >= D, GDN_ERR_INVALID, "%s: the output rows must be at least as long as the input rows", who);
    if (rows == 0) return GDN_OK;
    GDN_CHECK_ARG(x && y && rstd && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0, GDN_ERR_INVALID, "%s: NULL or unaligned tensor", who);
    return dtype == GDN_DTYPE_BF16 ? launch_l2norm<bf16_t>(x, y, rstd, nullptr, rows, 1, (int)D, (int)Dout, false, (hipStream_t)stream)
                                   : launch_l2norm<f16_t>(x, y, rstd, nullptr, rows, 1, (int)D, (int)Dout, false, (hipStream_t)stream);
}

extern "C" int gdn_l2norm_bwd(const void* dyh, const void* y, const float* rstd, void* dx, int64_t rows, int64_t G, int64_t Din,
                              int64_t Dout, int dtype, void* stream) {
    using namespace gdn;
    const char* who = "gdn_l2norm_bwd";
    if (int rc = l2_args_ok(who, rows, Din, Dout, dtype)) return rc;
    GDN_CHECK_ARG(G >= 1 && G <= 4096 && Dout <= Din, GDN_ERR_INVALID, "%s: bad group size or output rows longer than input rows", who);
    GDN_CHECK_ARG((y == nullptr) == (rstd == nullptr), GDN_ERR_INVALID, "%s: y and rstd go together", who);
    if (rows == 0) return GDN_OK;
    GDN_CHECK_ARG(dyh && dx && (uintptr_t)dyh % 16 == 0 && (uintptr_t)dx % 16 == 0 && (uintptr_t)y % 16 == 0, GDN_ERR_INVALID,
                  "%s: NULL or unaligned tensor", who);
    return dtype == GDN_DTYPE_BF16 ? launch_l2norm<bf16_t>(y, dx, (float*)rstd, dyh, rows, (int)G, (int)Din, (int)Dout, true, (hipStream_t)stream)
                                   : launch_l2norm<f16_t>(y, dx, (float*)rstd, dyh, rows, (int)G, (int)Din, (int)Dout, true, (hipStream_t)stream);
}
