// Error channel and version of the C ABI.
#include "gdn_common.h"
#include <algorithm>

namespace gdn {
static thread_local char g_err[512] = {0};
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
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
}  // namespace gdn

extern "C" int gdn_hip_abi_version(void) { return 5; }
extern "C" const char* gdn_last_error(void) { return gdn::g_err; }
