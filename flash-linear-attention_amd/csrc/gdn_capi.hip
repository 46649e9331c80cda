// Error channel and version of the C ABI.
#include "gdn_common.h"
#include <algorithm>
#include <mutex>
#include <unordered_map>

namespace gdn {
static thread_local char g_err[512] = {0};
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int ensure_dynamic_smem_for(const void* kernel, size_t bytes, const char* what) {
    static std::mutex lock;
    static std::unordered_map<const void*, SmemAttrDone> table;
    std::lock_guard<std::mutex> hold(lock);
    return ensure_dynamic_smem(kernel, bytes, table[kernel], what);
}

// dst = src (or zero when src is NULL), `count` floats, count a multiple of 4 and both 16-byte aligned or anything
// else element by element.  A kernel rather than a memset / memcpy node so that callers may capture it in a graph.
__global__ void state_copy_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t count) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) dst[i] = src ? src[i] : 0.f;
}

int launch_state_copy(const float* src, float* dst, int64_t count, hipStream_t stream) {
    if (count <= 0 || src == dst) return GDN_OK;
    const int64_t blocks = std::min<int64_t>((count + 255) / 256, 4096);
    hipLaunchKernelGGL(state_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, dst, count);
    return check_launch("state_copy_kernel");
}

// Calibration stream: every 64 KB block of `data` read, changed and written back in place by one workgroup of 256
// threads, with a workgroup-wide reduction between the last read and the first write - the memory traffic and the
// dependency of a decode step without its arithmetic.
__global__ __launch_bounds__(256) void calib_rmw_kernel(float* data, int64_t blocks, int xcd_run) {
    extern __shared__ char pad[];
    __shared__ f32x4 part[4][32];
    int64_t b = blockIdx.x;
    if (xcd_run > 0) {
        const int64_t s = b >> 3;
        b = ((s / xcd_run) * 8 + (b & 7)) * xcd_run + s % xcd_run;
    }
    if (b >= blocks) return;
    f32x4* base = (f32x4*)data + b * 4096 + threadIdx.x;
    f32x4 x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = __builtin_nontemporal_load(base + 256 * i);
    f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 16; ++i) s4 += x[i];
#pragma unroll
    for (int j = 0; j < 4; ++j) s4[j] += __shfl_xor(s4[j], 32, 64);
    const int c = threadIdx.x & 31, w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) < 32) part[w][c] = s4;
    __syncthreads();
    s4 = (part[0][c] + part[1][c] + part[2][c] + part[3][c]) * 1e-9f;
#pragma unroll
    for (int i = 0; i < 16; ++i) __builtin_nontemporal_store(x[i] + s4, base + 256 * i);
}
}  // namespace gdn

extern "C" int gdn_calib_rmw(float* data, int64_t n_floats, int xcd_run, int workgroups_per_cu, void* stream) {
    using namespace gdn;
    GDN_CHECK_ARG(data && n_floats > 0 && n_floats % 16384 == 0 && ((uintptr_t)data % 16) == 0, GDN_ERR_INVALID,
                  "gdn_calib_rmw: data must be 16-byte aligned and hold a multiple of 16384 floats");
    GDN_CHECK_ARG(xcd_run >= 0 && workgroups_per_cu >= 0 && workgroups_per_cu <= 8, GDN_ERR_INVALID, "gdn_calib_rmw: bad shape");
    const int64_t blocks = n_floats / 16384;
    const int64_t grid = xcd_run > 0 ? ((blocks + xcd_run - 1) / xcd_run + 7) / 8 * 8 * xcd_run : blocks;
    GDN_CHECK_ARG(grid < (1ll << 31), GDN_ERR_UNSUPPORTED, "gdn_calib_rmw: too many blocks");
    // unused LDS caps the workgroups that share a CU
    const size_t pad = workgroups_per_cu > 0 ? (size_t)(160 * 1024 / workgroups_per_cu - 8192) : 0;
    if (pad > 0 && hipFuncSetAttribute((const void*)calib_rmw_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pad) != hipSuccess)
        return check_launch("hipFuncSetAttribute(calib_rmw)");
    hipLaunchKernelGGL(calib_rmw_kernel, dim3((unsigned)grid), dim3(256), pad, (hipStream_t)stream, data, blocks, xcd_run);
    return check_launch("calib_rmw_kernel");
}

extern "C" int gdn_hip_abi_version(void) { return 13; }
extern "C" const char* gdn_last_error(void) { return gdn::g_err; }
