// Building blocks of the chunk kernels that keep their operands as row-major LDS tiles (the backward pass of the gated delta
// rule, the chunked KDA forward): where a chunk lies in a packed batch, tiles on their way from global memory through
// registers into LDS, matrix-core operand fragments read from such tiles, small cross-lane sums.
// A product's two operands have the same register layout (lane (c16, g) holds index c16 and the 8 contraction indices
// 8g .. 8g+7 of a 32-wide step), so there are just two ways to fetch an operand fragment from a row-major tile: `frag_rows`
// (the contraction runs along a row: one 16-byte read) and `frag_cols` (the contraction runs down a column: two transposing
// LDS reads).  The result of run(a, b) holds, in lane (c16, g), column c16 (b's index) and rows 4g .. 4g+3 (a's index).
#pragma once
#include "gdn_chunk_common.h"

namespace gdn {

constexpr int BD = 128;              // value columns of these kernels; key features: KD = 128 KT with KT = 1 or 2 (a template argument)
constexpr int P128 = BD + 8;         // LDS pitch, in elements, of a [64][128] tile ([64][KD] tiles: KD + 8)
constexpr int P64 = CH + 8;          // ... of a [64][64] tile
constexpr int PL = CH + 4;           // pitch of the fp32 matrix L


// Params types used with chunk_at / seq_at carry: cu_seqlens, chunk_table, chunk_offsets, flags, T, NT.
// ---- geometry ------------------------------------------------------------------------------
struct ChunkAt { int64_t tok0; int valid; };
template <typename P>
__device__ __forceinline__ ChunkAt chunk_at(const P& p, int64_t ci) {
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    if (p.cu_seqlens) {
        const int64_t n = load_index(p.chunk_table, 2 * ci, cu32), it = load_index(p.chunk_table, 2 * ci + 1, cu32);
        const int64_t bos = load_index(p.cu_seqlens, n, cu32), eos = load_index(p.cu_seqlens, n + 1, cu32);
        const int64_t t0 = bos + it * CH;
        return ChunkAt{t0, (int)min((int64_t)CH, eos - t0)};
    }
    // (32-bit: the entries refuse calls with 2^31 chunks or more, and a 64-bit division costs some hundred instructions)
    const uint32_t b = (uint32_t)ci / (uint32_t)p.NT, it = (uint32_t)ci - b * (uint32_t)p.NT;
    return ChunkAt{(int64_t)b * p.T + (int64_t)it * CH, (int)min((int64_t)CH, p.T - (int64_t)it * CH)};
}
// Unit u = chunk * HV + v-head of the kernels that walk over the units: its v-head, q/k head and chunk.  (32-bit arithmetic,
// as above: these kernels are bound by the rate at which one or two waves per SIMD issue instructions.)
struct UnitAt { int hv, hq; ChunkAt c; };
template <typename P>
__device__ __forceinline__ UnitAt unit_at(const P& p, int64_t u) {
    const uint32_t HV = (uint32_t)p.HV, ch = (uint32_t)u / HV, hv = (uint32_t)u - ch * HV, G = HV / (uint32_t)p.H;
    return UnitAt{(int)hv, (int)(G == 1 ? hv : hv / G), chunk_at(p, ch)};
}
struct SeqAt { int64_t bos, len, cbase, nc; };
template <typename P>
__device__ __forceinline__ SeqAt seq_at(const P& p, int64_t n) {
    const bool cu32 = p.flags & GDN_FLAG_CU_INT32;
    SeqAt s;
    if (p.cu_seqlens) {
        s.bos = load_index(p.cu_seqlens, n, cu32);
        s.len = load_index(p.cu_seqlens, n + 1, cu32) - s.bos;
        s.cbase = load_index(p.chunk_offsets, n, cu32);
    } else {
        s.bos = n * p.T; s.len = p.T; s.cbase = n * p.NT;
    }
    s.nc = (s.len + CH - 1) / CH;
    return s;
}

// ---- tiles ---------------------------------------------------------------------------------
// 64 rows of NCOLS elements from global memory (row r at g + r * stride; rows from `valid` on read as zero) into a
// row-major LDS tile, by all 256 threads.  Loads first, stores after: the loads of one tile are in flight together.
template <int NCOLS, typename T>
__device__ __forceinline__ void load_tile(T* s, int pitch, const T* g, int64_t stride, int valid, int tid) {
    constexpr int PPR = NCOLS / 8, TOTAL = 64 * PPR, N = (TOTAL + 255) / 256;
    u32x4 x[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const int idx = tid + 256 * i, row = idx / PPR, pc = idx % PPR;
        x[i] = u32x4{0u, 0u, 0u, 0u};
        if (idx < TOTAL && row < valid) x[i] = *(const u32x4*)(g + row * stride + pc * 8);
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const int idx = tid + 256 * i, row = idx / PPR, pc = idx % PPR;
        if (idx < TOTAL) *(u32x4*)(s + row * pitch + pc * 8) = x[i];
    }
}

// The same in two halves, for loops that fetch the next tile while they work on the current one.
template <int NCOLS, int NTH = 256>
struct TileRegs { u32x4 x[64 * (NCOLS / 8) >= NTH ? 64 * (NCOLS / 8) / NTH : 1]; };
template <int NCOLS, int NTH = 256, typename T>
__device__ __forceinline__ void fetch_tile(TileRegs<NCOLS, NTH>& r, const T* g, int64_t stride, int valid, int tid) {
    constexpr int PPR = NCOLS / 8, TOTAL = 64 * PPR, N = TOTAL >= NTH ? TOTAL / NTH : 1, RPI = NTH / PPR;      // a thread's pieces lie RPI rows apart
    static_assert(TOTAL % NTH == 0 || TOTAL < NTH, "whole rounds of the workgroup's threads, or less than one");
    const int row0 = tid / PPR, pc = tid % PPR;
    const char* at = (const char*)(g + (int64_t)row0 * stride + pc * 8);
    const int64_t step = (int64_t)RPI * stride * (int64_t)sizeof(T);
    if (valid >= 64 && TOTAL >= NTH) {                          // (the same for the whole workgroup) full chunk: plain loads
#pragma unroll
        for (int i = 0; i < N; ++i) r.x[i] = *(const u32x4*)(at + i * step);
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            r.x[i] = u32x4{0u, 0u, 0u, 0u};
            if (row0 + RPI * i < valid && tid < TOTAL) r.x[i] = *(const u32x4*)(at + i * step);
        }
    }
}
template <int NCOLS, int NTH = 256, typename T>
__device__ __forceinline__ void put_tile(T* s, int pitch, const TileRegs<NCOLS, NTH>& r, int tid) {
    constexpr int PPR = NCOLS / 8, TOTAL = 64 * PPR, N = TOTAL >= NTH ? TOTAL / NTH : 1, RPI = NTH / PPR;
    T* at = s + (tid / PPR) * pitch + (tid % PPR) * 8;
    if (TOTAL < NTH && tid >= TOTAL) return;
#pragma unroll
    for (int i = 0; i < N; ++i) *(u32x4*)(at + i * RPI * pitch) = r.x[i];
}
// ROWS rows of NCOLS elements of an LDS tile out to global memory (row r at g + r * stride), 16 bytes a lane along the rows:
// whole cache lines per group of lanes, where the lanes that hold a result as matrix-instruction output would write 8-byte pieces.
// (`valid`: rows from there on are left alone)
template <int ROWS, int NCOLS, int NTH, typename T>
__device__ __forceinline__ void copy_rows_out(T* g, int64_t stride, const T* s, int pitch, int tid, int valid = ROWS) {
    constexpr int PPR = NCOLS / 8, TOTAL = ROWS * PPR, N = TOTAL / NTH;
    static_assert(TOTAL % NTH == 0, "whole rounds of the workgroup's threads");
    u32x4 x[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const int idx = tid + NTH * i;
        x[i] = *(const u32x4*)(s + (idx / PPR) * pitch + (idx % PPR) * 8);
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const int idx = tid + NTH * i;
        if (idx / PPR < valid) *(u32x4*)(g + (int64_t)(idx / PPR) * stride + (idx % PPR) * 8) = x[i];
    }
}
// operand fragment whose contraction runs along a row: index r0 + c16, contraction c0 + 8g + e
template <typename T>
__device__ __forceinline__ typename Mma<T>::V8 frag_rows(const T* s, int pitch, int r0, int c0, int lane) {
    return *(const typename Mma<T>::V8*)(s + (r0 + (lane & 15)) * pitch + c0 + 8 * (lane >> 4));
}
// operand fragment whose contraction runs down a column: index c0 + c16, contraction r0 + 8g + e
template <typename T>
__device__ __forceinline__ typename Mma<T>::V8 frag_cols(const T* s, int pitch, int r0, int c0, int lane) {
    const int a = lane & 15;
    const T* at = s + (r0 + 8 * (lane >> 4) + (a >> 2)) * pitch + c0 + 4 * (a & 3);
    return join<typename Mma<T>::V8>(Mma<T>::tr_read(at), Mma<T>::tr_read(at + 4 * pitch));
}
template <typename T>
__device__ __forceinline__ typename Mma<T>::V4 pack4(f32x4 x) {
    return typename Mma<T>::V4{(T)x[0], (T)x[1], (T)x[2], (T)x[3]};
}
__device__ __forceinline__ float sum_over_g(float x) {          // over the four lanes that share c16
    x += __shfl_xor(x, 16, 64);
    return x + __shfl_xor(x, 32, 64);
}
__device__ __forceinline__ float sum_over_c16(float x) {        // over the sixteen lanes that share g
    x += __shfl_xor(x, 1, 64); x += __shfl_xor(x, 2, 64); x += __shfl_xor(x, 4, 64);
    return x + __shfl_xor(x, 8, 64);
}
// x summed over the four lanes of a quad (lanes 4n .. 4n+3), in every one of them
__device__ __forceinline__ float sum_over_quad(float x) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));   // [2,3,0,1]
}
#define ZERO4 (f32x4{0.f, 0.f, 0.f, 0.f})


// A = (I + L)^-1 for a strictly lower triangular 64 x 64 L, by forward substitution in fp32:
// A[i][c] = [i == c] - sum_{j < i} L[i][j] A[j][c].  Four waves, wave w the columns 16w .. 16w+15: a quad of lanes per
// column c, lane gq of the quad keeps A[j][c] for j = gq mod 4 and adds up its part of the sum.  sL holds entry (i, j)
// at [i][j % 4][j / 4] (pitch PL; zeros from the diagonal on within the 16 x 16 diagonal blocks); A goes to sA (pitch
// P64) in the operand type.  The caller's barriers separate it from the writers of sL and the readers of sA.
template <typename T>
__device__ __forceinline__ void solve_unit_lower(const float* sL, T* sA, int w, int lane) {
    const int c = 16 * w + (lane >> 2), gq = lane & 3;
    float a[16];
#pragma unroll
    for (int m = 0; m < 16; ++m) a[m] = 0.f;
#pragma unroll
    for (int i = 0; i < 64; ++i) {
        float part0 = 0.f, part1 = 0.f;
#pragma unroll
        for (int m4 = 0; 16 * m4 < i; ++m4) {                   // entries j = 4m + gq < i; those from i on are stored as zeros
            const f32x4 l = *(const f32x4*)(sL + i * PL + gq * 16 + 4 * m4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (4 * (4 * m4 + e) < i) {
                    if (e & 1) part1 += l[e] * a[4 * m4 + e];
                    else part0 += l[e] * a[4 * m4 + e];
                }
            }
        }
        const float ai = (i == c ? 1.f : 0.f) - sum_over_quad(part0 + part1);
        if (gq == (i & 3)) { a[i >> 2] = ai; sA[i * P64 + c] = (T)ai; }
    }
}

// The same inverse by blocks of 16, for the same four waves (all of them must call it: it holds two barriers).  Wave a first
// inverts the diagonal block a on its own (X_a (I + L_aa) = I by rows from the right: lane c16 owns row c16, 16 short steps
// without any exchange between lanes) and leaves X_a in LDS; then wave b computes block column b of A from
//     A_bb = X_b,   A_ab = -X_a sum_{b <= m < a} L_am A_mb   (a > b)
// on the matrix cores in fp32 (v_mfma_f32_16x16x4_f32): the left factors L_am and X_a come from LDS, the right factors are
// the blocks just computed, which an accumulator holds in the layout a right factor needs.  64 dependent steps become 16
// plus at most nine 16 x 16 products.  sX: 1024 floats of scratch, which may be the memory of sA itself.
template <typename T>
__device__ __forceinline__ void solve_unit_lower_blocks(const float* sL, float* sX, T* sA, int w, int lane) {
    const int c16 = lane & 15, g = lane >> 4;
    {
        float x[16], acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int i = 15; i >= 0; --i) {
            x[i] = ((i == c16) ? 1.f : 0.f) - acc[i];
            // row i of the diagonal block: entry j = 4q + e at [e][4w + q]
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (e >= i) continue;
                const f32x4 l = *(const f32x4*)(sL + (16 * w + i) * PL + e * 16 + 4 * w);
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (4 * q + e < i) acc[4 * q + e] += l[q] * x[i];
            }
        }
        if (g == 0) {
#pragma unroll
            for (int q = 0; q < 4; ++q) *(f32x4*)(sX + w * 256 + c16 * 16 + 4 * q) = f32x4{x[4 * q], x[4 * q + 1], x[4 * q + 2], x[4 * q + 3]};
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    f32x4 A[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        A[a] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (a < w) continue;
        if (a == w) {
            const float* t = sX + a * 256;
            A[a] = f32x4{t[(4 * g) * 16 + c16], t[(4 * g + 1) * 16 + c16], t[(4 * g + 2) * 16 + c16], t[(4 * g + 3) * 16 + c16]};
            continue;
        }
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < a; ++m) {
            if (m < w) continue;
            // left factor L_am by rows: entry (16a + c16, 16m + 4g + e) at [e][4m + g]
#pragma unroll
            for (int e = 0; e < 4; ++e)
                t = __builtin_amdgcn_mfma_f32_16x16x4f32(sL[(16 * a + c16) * PL + e * 16 + 4 * m + g], A[m][e], t, 0, 0, 0);
        }
        const f32x4 xa = *(const f32x4*)(sX + a * 256 + c16 * 16 + 4 * g);
        f32x4 r = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; ++e) r = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[e], t[e], r, 0, 0, 0);
        A[a] = -r;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");     // (every wave has read the X tiles: sA may take their place)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int r = 0; r < 4; ++r) sA[(16 * a + 4 * g + r) * P64 + 16 * w + c16] = (T)A[a][r];
}

}  // namespace gdn
