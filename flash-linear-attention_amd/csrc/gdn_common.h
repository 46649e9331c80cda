// Shared helpers for the gfx950 gated-delta-rule kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/gdn_hip.h"

namespace gdn {

void set_error(const char* fmt, ...);
// dst = src, or zero when src is NULL (`count` floats), as a kernel on `stream`
int launch_state_copy(const float* src, float* dst, int64_t count, hipStream_t stream);

#define GDN_CHECK_ARG(cond, code, ...)            \
    do {                                          \
        if (!(cond)) {                            \
            gdn::set_error(__VA_ARGS__);          \
            return (code);                        \
        }                                         \
    } while (0)

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(e));
        return GDN_ERR_LAUNCH;
    }
    return GDN_OK;
}

// Raises the dynamic LDS limit of a kernel once per device (the attribute belongs to the function on
// the current device; a process may drive several).  `done` is a per-kernel table owned by the caller.
struct SmemAttrDone { bool dev[64] = {}; };
inline int ensure_dynamic_smem(const void* kernel, size_t bytes, SmemAttrDone& done, const char* what) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return check_launch(what);
    const bool tracked = dev >= 0 && dev < 64;
    if (tracked && done.dev[dev]) return GDN_OK;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return check_launch(what);
    if (tracked) done.dev[dev] = true;
    return GDN_OK;
}

// The same for launchers that pick among many kernels at run time: the table is kept here, one entry per kernel.
int ensure_dynamic_smem_for(const void* kernel, size_t bytes, const char* what);

// ---- element types -------------------------------------------------------
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x) { return (T)x; }

// g/beta may arrive in any float type; they are tiny, so a run-time switch is enough.
__device__ __forceinline__ float load_scalar(const void* p, int64_t i, int dtype) {
    if (dtype == GDN_DTYPE_F32) return ((const float*)p)[i];
    if (dtype == GDN_DTYPE_BF16) return (float)((const bf16_t*)p)[i];
    return (float)((const f16_t*)p)[i];
}

// The same number as raw bits (16-bit types in the low half), to be converted where it is used: a load whose result is
// converted on the spot makes the wave wait there for it and for every load requested before it, which undoes a prefetch.
__device__ __forceinline__ uint32_t load_scalar_bits(const void* p, int64_t i, int dtype) {
    if (dtype == GDN_DTYPE_F32) return ((const uint32_t*)p)[i];
    return ((const uint16_t*)p)[i];
}
__device__ __forceinline__ float scalar_of_bits(uint32_t bits, int dtype) {
    if (dtype == GDN_DTYPE_F32) return __builtin_bit_cast(float, bits);
    if (dtype == GDN_DTYPE_BF16) return __builtin_bit_cast(float, bits << 16);
    return (float)__builtin_bit_cast(f16_t, (uint16_t)bits);
}

__device__ __forceinline__ int64_t load_index(const void* p, int64_t i, bool is_i32) {
    return is_i32 ? (int64_t)((const int32_t*)p)[i] : ((const int64_t*)p)[i];
}

__device__ __forceinline__ float softplus_f(float x) {
    // log(1 + e^x) with the usual linear tail (torch threshold 20)
    return x > 20.f ? x : log1pf(__expf(x));
}

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + __expf(-x)); }
// The same with the hardware reciprocal (1 ulp) and base-2 exponential: for the streaming kernels, where the
// activation is most of the arithmetic per byte and the result is rounded to 16 bits anyway.
__device__ __forceinline__ float sigmoid_stream(float x) {
    return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// Asynchronous copy of 64 x 16 bytes from global memory straight into LDS: lane l fetches the
// 16 bytes at gbase + voff (gbase wave-uniform, voff per lane) and they land at the
// wave-uniform LDS byte offset `lds_off` + 16 l.  Issued from inline assembly on purpose: the
// compiler then keeps no account of it, and completion is awaited explicitly with s_waitcnt
// vmcnt before the barrier that publishes the data.
__device__ __forceinline__ void gather_1k_to_lds(const char* gbase, uint32_t voff, uint32_t lds_off) {
    lds_off = __builtin_amdgcn_readfirstlane(lds_off);          // wave-uniform by construction; make them scalars
    const uint64_t g = (uint64_t)gbase;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)g), hi = __builtin_amdgcn_readfirstlane((uint32_t)(g >> 32));
    const uint64_t gs = ((uint64_t)hi << 32) | lo;
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_off), "v"(voff), "s"(gs));
}

// The same copy for the lanes named by `mask` only (the others leave their 16 bytes of LDS as they are).
// The instruction is issued whatever the mask, so counts of outstanding operations do not depend on it.
__device__ __forceinline__ void gather_1k_to_lds_masked(const char* gbase, uint32_t voff, uint32_t lds_off, uint64_t mask) {
    lds_off = __builtin_amdgcn_readfirstlane(lds_off);
    const uint64_t g = (uint64_t)gbase;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)g), hi = __builtin_amdgcn_readfirstlane((uint32_t)(g >> 32));
    const uint64_t gs = ((uint64_t)hi << 32) | lo;
    const uint32_t mlo = __builtin_amdgcn_readfirstlane((uint32_t)mask), mhi = __builtin_amdgcn_readfirstlane((uint32_t)(mask >> 32));
    mask = ((uint64_t)mhi << 32) | mlo;                         // wave-uniform by construction; make it scalar registers
    uint64_t saved;
    asm volatile("s_mov_b32 m0, %1\n\t"
                 "s_and_saveexec_b64 %0, %4\n\t"
                 "global_load_lds_dwordx4 %2, %3\n\t"
                 "s_mov_b64 exec, %0"
                 : "=&s"(saved) : "s"(lds_off), "v"(voff), "s"(gs), "s"(mask) : "scc");
}

template <int N>
__device__ __forceinline__ void wait_vm_at_most() {
    static_assert(N >= 0 && N <= 63, "the vector-memory counter has 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// Workgroup barrier that only waits for this wave's LDS traffic.  __syncthreads() also drains
// the vector-memory counter, which would serialise the global prefetch of later chunks
// behind every barrier of the current one.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

}  // namespace gdn
