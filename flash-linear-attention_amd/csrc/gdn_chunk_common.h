// Definitions shared by the chunked-prefill kernels (gfx950, 64-token chunks, K = V = 128).
//
// MFMA register layout used throughout (wave64, lane l, c16 = l%16, g = l/16):
//   A operand (M x 32): lane holds row c16, 8 contraction indices chosen by g;
//   B operand (32 x N): lane holds column c16, the same 8 contraction indices;
//   C/D (16 x 16):      lane holds column c16, rows 4g..4g+3.
// Any assignment of contraction indices to (g, element) is valid as long as A and B agree.
// The scan kernels use {16a+4g+r} U {16b+4g+r} for a pair of 16-row tiles (a, b): that is
// exactly how a C/D result is spread over lanes, so an accumulator can be converted in
// place into the B operand of the next product, and swapping the two operands of an MFMA
// yields the transposed tile.
#pragma once
#include "gdn_common.h"
#include <type_traits>
#include <algorithm>

namespace gdn {

constexpr int CH = 64;                       // chunk length
constexpr float RCP_LN2_F = 1.4426950216f;   // fla/ops/utils/constant.py:10

typedef bf16x4 __attribute__((address_space(3)))* lds_bf16x4_ptr;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef s16x4 __attribute__((address_space(3)))* lds_s16x4_ptr;

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    typedef bf16x8 V8;
    typedef bf16x4 V4;
    static __device__ __forceinline__ f32x4 run(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    // LDS transpose read: the 16 lanes of a group each pass the address of 4 consecutive
    // elements; lane L receives element L%4 of the runs addressed by lanes L/4, L/4+4, L/4+8, L/4+12.
    static __device__ __forceinline__ V4 tr_read(const bf16_t* p) {
        return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)p);
    }
};
template <> struct Mma<f16_t> {
    typedef f16x8 V8;
    typedef f16x4 V4;
    static __device__ __forceinline__ f32x4 run(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ V4 tr_read(const f16_t* p) {
        return __builtin_bit_cast(f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p));
    }
};

template <typename V8, typename V4>
__device__ __forceinline__ V8 join(V4 a, V4 b) {
    return V8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
}

// 2^x as a single v_exp_f32 (results below 2^-126 flush to zero, which is what a decay wants)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Per-chunk workspace written by the prepare kernel (element counts for K = V = 128):
//   Tab fp32 [NC][HV][256]                  [0..63] 2^(G_last-G_t), [64..127] scale*2^G_t, [128] G_last (log2 units)
//   Wf  T    [NC][HV][4 tt][4 s][64][8]     w rows of t-tile tt, key tiles (2s, 2s+1)
//   Uf  T    [NC][HV][8 n ][4 tt][64][4]    u, C/D layout of tile (t-tile tt, value tile n)
//   Pf  T    [NC][HV][4 tt][2 s][64][8]     scale*P rows of t-tile tt, t-tiles (2s, 2s+1) as columns
//   KTf T    [NC][H ][8 m ][2 s][64][8]     k^T rows of key tile m, t-tiles (2s, 2s+1)
//   Qf  T    [NC][H ][4 tt][4 s][64][8]     q rows of t-tile tt, key tiles (2s, 2s+1)
struct ChunkWs {
    float* Seg;          // 3 * seg_slots 128x128 fp32 matrices for the segment-parallel scan
    float* Tab;
    void* Wf;
    void* Uf;
    void* Pf;
    void* KTf;
    void* Qf;
};
constexpr int64_t WS_TAB = 256, WS_W = 8192, WS_U = 8192, WS_P = 4096, WS_KT = 8192, WS_Q = 8192;   // elements per (chunk, head)

constexpr int64_t SEG_SLOTS_MAX = 640;            // upper bound on (sequences * heads * segments) when segmenting

inline size_t ws_align(size_t x) { return (x + 255) & ~(size_t)255; }

inline size_t ws_layout(int64_t NC, int64_t H, int64_t HV, char* base, ChunkWs* ws) {
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += ws_align(bytes); return base ? (void*)(base + o) : nullptr; };
    const size_t seg_slots = (size_t)std::min<int64_t>((NC * HV + 3) / 4, SEG_SLOTS_MAX);
    void* Seg = take(3 * seg_slots * 16384 * 4);
    void* Tab = take((size_t)NC * HV * WS_TAB * 4);
    void* Wf = take((size_t)NC * HV * WS_W * 2);
    void* Uf = take((size_t)NC * HV * WS_U * 2);
    void* Pf = take((size_t)NC * HV * WS_P * 2);
    void* KTf = take((size_t)NC * H * WS_KT * 2);
    void* Qf = take((size_t)NC * H * WS_Q * 2);
    if (ws) { ws->Seg = (float*)Seg; ws->Tab = (float*)Tab; ws->Wf = Wf; ws->Uf = Uf; ws->Pf = Pf; ws->KTf = KTf; ws->Qf = Qf; }
    return off;
}

struct ChunkParams {
    const void* q; const void* k; const void* v; const void* g; const void* beta;
    const float* h0; float* ht; void* o;
    const void* cu_seqlens; const void* chunk_table; const void* chunk_offsets;
    ChunkWs ws;
    int64_t T; int H, HV; int64_t N; int64_t NT;       // NT: chunks per sequence (dense input)
    float scale; int gb_dtype; uint32_t flags;
    int nslab; int64_t NH;
};

// Workgroup barrier that only waits for this wave's LDS traffic.  __syncthreads() also drains
// the vector-memory counter, which would serialise the global prefetch of later chunks
// behind every barrier of the current one.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 8-byte global store issued from inline assembly.  The compiler's wait-count bookkeeping
// does not see it, so the prefetched loads of the scan loop stay the only operations it
// counts and it can wait for "all but the newest N loads" instead of draining the queue
// (loads and stores share one hardware counter, and once both are pending the compiler
// falls back to waiting for everything).  The extra, uncounted stores only make the
// hardware counter larger than the compiler assumes, i.e. its waits err on the late side.
__device__ __forceinline__ void store_b64_uncounted(void* ptr, u32x2 data) {
    asm volatile("global_store_dwordx2 %0, %1, off" : : "v"(ptr), "v"(data) : "memory");
}

// 16x16 product of fp32 matrices held in LDS on the fp32 matrix cores:
// C = A[16 x 4*nk] * B[4*nk x 16]; result in C/D layout.
__device__ __forceinline__ f32x4 mm16_f32(const float* A, int lda, const float* B, int ldb, int nk, int c16, int g) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < nk; ++kk) {
        const float a = A[c16 * lda + 4 * kk + g];
        const float b = B[(4 * kk + g) * ldb + c16];
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc, 0, 0, 0);
    }
    return acc;
}


// Segment-parallel evaluation of long dense sequences: every sequence is cut into `nseg`
// segments of `seg_chunks` chunks; per (sequence, head, segment) the buffers hold 128x128 fp32
// matrices ([K][V], K-first): sloc = state reached from a zero state (segment 0: from the true
// initial state), mseg = transition matrix, sin = merged state at the start of the segment.
struct SegmentPlan {
    int kind;
    int nseg;
    int seg_chunks;
    float* sloc;
    float* mseg;
    float* sin;
};

// launchers defined next to their kernels
template <typename T> int launch_prepare(const ChunkParams& p, int64_t num_chunks, hipStream_t stream);
template <typename T> int launch_scan_slab(const ChunkParams& p, hipStream_t stream);
template <typename T> int launch_scan_wide(const ChunkParams& p, hipStream_t stream);
template <typename T> int launch_scan_segments(const ChunkParams& p, SegmentPlan sp, hipStream_t stream);

}  // namespace gdn
