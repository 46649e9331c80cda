// Definitions shared by the chunked-prefill kernels (gfx950, 64-token chunks, K = V = 128).
//
// MFMA register layout used throughout (wave64, lane l, c16 = l%16, g = l/16):
//   A operand (M x 32): lane holds row c16, 8 contraction indices chosen by g;
//   B operand (32 x N): lane holds column c16, the same 8 contraction indices;
//   C/D (16 x 16):      lane holds column c16, rows 4g..4g+3.
// Any assignment of contraction indices to (g, element) is valid as long as A and B agree.
// The scan kernel uses {16a+4g+r} U {16b+4g+r} for a pair of 16-row tiles (a, b): that is
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

// Workspace record written by the prepare kernel per (chunk, v-head): 12 KB in 1 KB pieces that the scan
// copies verbatim into LDS.  Xb and P are stored as matrix-core operand fragments
// ([lane][8]): rows of t-tile tt, columns t' in {32sp+4g+r} U {32sp+16+4g+r}.  Both are
// lower triangular: the fragments (tt, sp) = (0,1), (1,1) are identically zero and are not
// stored, and of (0,0), (2,1) only the first half (4 values per lane) is.
//   Xb   T    5 KB        (I+L)^-1 diag(beta)
//   P    T    5 KB        scale * tril(q k^T 2^(G_t-G_t')): room only.  Every scan kernel forms P itself, from its q and k
//                         tiles and the second table, into this place of its LDS copy; the prepare kernel writes it to
//                         memory on request (GDN_FLAG_RECORD_P), for callers that look at the records
//   tab  fp32 [256]       [0..63] 2^(G_last-G_t), [64..127] scale*2^G_t, [128..191] 2^G_t, [192] G_last (log2 units),
//                         the first and the third times the row factor 1/|k_t| of the l2 normalisation
//   tab2 fp32 [256]       [0..63] G_t (log2 units), [64..127] scale, [128..191] 1/|k_t|: what P needs
// The row factors 1/|q_t| of the l2 normalisation are not in the records: the prepare kernel does not read q.  The scan
// kernels take them from the q tiles in LDS where they form P (row_rnorm below), scale P with them and multiply them
// into [64..127] of their LDS copy of `tab` before anything reads it.  (Not always: see FLAG_Q_NORM_IN_SCAN; without it the
// prepare kernel reads q for its norms and both tables carry 1/|q_t|, scale/|q_t|.)
constexpr int REC_X = 0, REC_P = 5120, REC_TAB = 10240, REC_TAB2 = 11264;
constexpr int64_t REC_BYTES = 12288;
constexpr int REC_PIECES_X = 5, REC_PIECES_P = 5, REC_PIECE_TAB = 10, REC_PIECE_TAB2 = 11;      // in 1 KB pieces: Xb = 0..4, P = 5..9, tab = 10, tab2 = 11
constexpr int TAB_DEC = 0, TAB_SG = 64, TAB_EG = 128, TAB_GLAST = 192;
constexpr int TAB2_G = 0, TAB2_NQS = 64, TAB2_NK = 128;
// Who applies the row factors 1/|q_t| of the in-kernel l2 norm (a bit of ChunkParams::flags that the entry points set, above
// the caller's flags): the scan kernels, which have q in LDS anyway - except for head dims up to 64 (the scan's step is short
// and P is on its critical path) and for wide keys on few units (every 64-column workgroup of a head would form the norms
// again, while a prepare kernel that does not fill the chip reads q for nothing).
constexpr uint32_t FLAG_Q_NORM_IN_SCAN = 1u << 30;
inline bool q_norm_in_scan(uint32_t flags, int64_t K, int64_t V, int64_t units) {
    if (!(flags & GDN_FLAG_QK_L2NORM) || (K <= 64 && V <= 64)) return false;
    return K <= 128 || units >= 4096;
}
// 1/|q_t| of the token row that this lane's q fragments belong to (lane (c16, g) holds 8 features per fragment of row c16
// of a t-tile).  On the matrix cores: the tile's q q^T, whose diagonal element (c16, c16) lands in lane (c16, g = c16 / 4),
// register c16 % 4, and is handed to the other three lanes of the row by one cross-lane read.
template <typename T, int N>
__device__ __forceinline__ float row_rnorm(const typename Mma<T>::V8 (&qb)[N], int c16) {
    f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < N; ++i) d = Mma<T>::run(qb[i], qb[i], d);
    const int r = c16 & 3;
    const float own = r == 0 ? d[0] : r == 1 ? d[1] : r == 2 ? d[2] : d[3];
    return rsqrtf(__shfl(own, 16 * (c16 >> 2) + c16, 64) + 1e-6f);
}
// Besides the records the prepare kernel leaves one number per (chunk, v-head): an upper bound, in log2 units, on how much
// the chunk's transition S -> 2^G_last S - k~^T (Xb 2^G k) S can stretch any state:
//   bound = sum_t [ log2 gamma_t + log2 max(1, |1 - beta_t |k_t|^2|) ]      (each token's factor gamma_t (I - beta_t k_t k_t^T))
// A run of chunks whose bounds add up to at most WARM_LOG2 forgets what came before it to within 2^WARM_LOG2 of that
// state's size: the state in front of the run would have to be 2^8 times the size of the state behind it for the
// dropped part to reach the rounding of the fp32 state (2^-24 of its own size), and 2^24 times its size to reach the
// operator's error bar (5e-3, set by the 16-bit operands).  So a time segment may start from a ZERO state that many
// chunks early instead of from the exact state that a first pass and a merge would have to compute.  (Measured against
// -48: warm-ups a third shorter, config 3 0.317 instead of 0.32 ms; with wide keys, where a head that cannot start warm is
// evaluated whole, more heads qualify: the forward of the layer's default shape with a random A_log 0.5 instead of 1.95 ms.
// -24 would take config 3 to 0.304 ms and leave no margin over the fp32 rounding.)
constexpr float WARM_LOG2 = -32.f;
constexpr int WARM_CAP_MAX = 64;
__host__ __device__ constexpr int p_slot(int tt, int sp) { return tt < 2 ? tt : 2 + 2 * (tt - 2) + sp; }
__host__ __device__ constexpr bool frag_half(int tt, int sp) { return (tt == 0 && sp == 0) || (tt == 2 && sp == 1); }
__host__ __device__ constexpr int frag_off(int tt, int sp) {          // bytes from the start of Xb or P
    return p_slot(tt, sp) == 0 ? 0 : p_slot(tt, sp) == 1 ? 512 : p_slot(tt, sp) == 2 ? 1536 : p_slot(tt, sp) == 3 ? 2560
         : p_slot(tt, sp) == 4 ? 3072 : 4096;
}
template <typename T>
__device__ __forceinline__ typename Mma<T>::V8 load_frag(const char* m, int tt, int sp, int lane) {
    typedef typename Mma<T>::V8 V8;
    typedef typename Mma<T>::V4 V4;
    if (frag_half(tt, sp)) {
        const V4 a = *(const V4*)(m + frag_off(tt, sp) + lane * 8);
        const T z = (T)0.f;
        return V8{a[0], a[1], a[2], a[3], z, z, z, z};
    }
    return *(const V8*)(m + frag_off(tt, sp) + lane * 16);
}
template <typename T>
__device__ __forceinline__ void store_frag(char* m, int tt, int sp, int lane, typename Mma<T>::V8 f) {
    typedef typename Mma<T>::V4 V4;
    if (frag_half(tt, sp)) *(V4*)(m + frag_off(tt, sp) + lane * 8) = V4{f[0], f[1], f[2], f[3]};
    else *(typename Mma<T>::V8*)(m + frag_off(tt, sp) + lane * 16) = f;
}

struct ChunkWs {
    float* Seg;          // 3 * seg_slots 128x128 fp32 matrices for the segment-parallel scan
    float* Bound;        // [NC][HV] log2 bound on the norm of every chunk's transition
    char* Rec;           // [NC][HV] records
};


constexpr int64_t SEG_SLOTS_MAX = 640;            // upper bound on (sequences * heads * segments) when segmenting

inline size_t ws_align(size_t x) { return (x + 255) & ~(size_t)255; }

// Number of time segments the sequential stage cuts every sequence into (0: whole sequences, one
// workgroup per sequence and head).  With few (sequence, head) runs and long dense sequences, time is
// cut so that every CU has a workgroup - never more workgroups than CUs: a second round of workgroups
// costs more than longer segments do.  Segments hold 8 chunks or more each (every pass also pays for
// filling and draining its pipeline and for a launch).  Two segments pay where they may start warm
// (one pass over half the chunks plus the warm-up); with exact start states only (first pass, merge,
// second pass) it takes three.  Either way the steps saved per workgroup must outweigh a warm-up of typical
// length plus the two launches that find nothing to do: 24 chunks or more.  Shared by the workspace size and the launch.
inline int plan_segments(int64_t N, int64_t HV, int64_t NT, int64_t num_chunks, bool dense, uint32_t flags) {
    const int64_t NH = N * HV;
    int nseg = 0;
    if (dense && NH > 0) {
        // (GDN_FLAG_SCAN_SEGMENTS asks for segments wherever they are possible at all: segments of 4 chunks)
        nseg = (int)std::min<int64_t>(256 / NH, NT / ((flags & GDN_FLAG_SCAN_SEGMENTS) ? 4 : 8));
        while (nseg > 0 && ((int64_t)nseg * NH > SEG_SLOTS_MAX || (int64_t)nseg * NH > (num_chunks * HV + 3) / 4)) --nseg;
    }
    bool segments = nseg >= ((flags & GDN_FLAG_SCAN_NO_WARM) ? 3 : 2) && NT - NT / std::max(nseg, 1) >= 24;
    if (flags & GDN_FLAG_SCAN_WIDE) segments = false;
    if ((flags & GDN_FLAG_SCAN_SEGMENTS) && nseg >= 2) segments = true;
    return segments ? nseg : 0;
}

// Wide keys (128 < K <= 256): a workgroup owns 64 value columns of a (sequence, value head) for all key rows, and time
// is cut into segments where whole sequences leave CUs without a workgroup: never more workgroups than CUs, segments of
// 8 chunks or more, and at least 24 chunks saved per workgroup (a warm-up of typical length must pay).  1 = whole sequences.
constexpr int W2_VB = 64;                                 // value columns per workgroup
constexpr int W2_KD = 256;                                // key rows of the segment matrices
inline int plan_segments256(int64_t N, int64_t H, int64_t HV, int64_t V, int64_t NT, bool dense, uint32_t flags) {
    const int64_t runs = N * HV * ((V + W2_VB - 1) / W2_VB);
    if (!dense || (flags & GDN_FLAG_SCAN_WIDE) || runs <= 0) return 1;
    int nseg = (int)std::min<int64_t>(256 / runs, NT / ((flags & GDN_FLAG_SCAN_SEGMENTS) ? 4 : 8));
    while (nseg >= 2 && (int64_t)nseg * N * HV > SEG_SLOTS_MAX) --nseg;
    if (nseg >= 2 && ((flags & GDN_FLAG_SCAN_SEGMENTS) || NT - NT / nseg >= 24)) return nseg;
    return 1;
}
// floats per (sequence, value head, segment) of the wide-key segment matrices: S_loc and S_in [256][VP], M [256][256]
__host__ __device__ inline size_t seg256_floats(int64_t V) {
    const size_t VP = (size_t)((V + W2_VB - 1) / W2_VB) * W2_VB;
    return 2 * (size_t)W2_KD * VP + (size_t)W2_KD * W2_KD;
}

// Workspace: the segment matrices (S_loc, M, S_in per (sequence, head, segment); none without segments),
// the transition bounds, then the records.  `seg_floats`: floats per slot (3 matrices of 128 x 128 by default).
inline size_t ws_layout(int64_t NC, int64_t HV, int64_t seg_slots, char* base, ChunkWs* ws, size_t seg_floats = 3 * 16384) {
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += ws_align(bytes); return base ? (void*)(base + o) : nullptr; };
    void* Seg = take((size_t)seg_slots * seg_floats * 4);
    void* Bound = take((size_t)NC * HV * 4);
    void* Rec = take((size_t)NC * HV * REC_BYTES);
    if (ws) { ws->Seg = (float*)Seg; ws->Bound = (float*)Bound; ws->Rec = (char*)Rec; }
    return off;
}

struct ChunkParams {
    const void* q; const void* k; const void* v; const void* g; const void* beta;
    const float* A_log; const float* dt_bias;     // optional gate activation (per value head)
    const float* h0; float* ht; void* o;
    const void* cu_seqlens; const void* chunk_table; const void* chunk_offsets;
    ChunkWs ws;
    int64_t T; int H, HV; int64_t N; int64_t NT;       // NT: chunks per sequence (dense input)
    int K, V;                                          // head dims of the caller's tensors (multiples of 8; K, V <= 128, or 128 < K <= 256 with any V)
    float scale; int gb_dtype; uint32_t flags;
    int64_t NH;
    int want_P;                                        // the prepare kernel also writes P (GDN_FLAG_RECORD_P)
};

// kind of run
constexpr int WIDE_WHOLE = 0;     // whole sequences, user h0 -> o, ht
constexpr int WIDE_PASS1 = 1;     // per segment: S_loc / M into the segment buffers
constexpr int WIDE_PASS2 = 2;     // per segment: from merged S_in -> o (last segment also ht)

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
    const float* bound;     // non-NULL: segments may start early from a zero state where the bounds allow it
    int warm_cap;           // ... at most this many chunks early (<= WARM_CAP_MAX)
};

// How many chunks before chunk it0 a run of (sequence, head) must start from a zero state so that at it0 it has
// forgotten the difference to the true state: the shortest run of chunks ending at it0 - 1 whose bounds add up to
// WARM_LOG2 or less.  When the start of the sequence comes first (within `cap` chunks) the answer is it0: the run
// starts at chunk 0 from the true initial state and is exact.  -1: not within `cap` chunks.  `bound` points at the
// entry of chunk 0 of the sequence for this head; entries of consecutive chunks are HV apart.  Lane l looks at
// chunk it0 - 1 - l; the result is the same in every lane.
__device__ __forceinline__ float warm_load(const float* bound, int HV, int64_t it0, int cap, int lane) {
    return (lane < cap && lane < it0) ? bound[(it0 - 1 - lane) * HV] : 0.f;
}
__device__ __forceinline__ int warm_from(float x, int64_t it0, int cap, int lane) {
    const bool in = lane < cap && lane < it0;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float y = __shfl_up(x, off, 64);
        if (lane >= off) x += y;
    }
    const uint64_t hit = __builtin_amdgcn_ballot_w64(in && x <= WARM_LOG2);
    if (hit) return __builtin_ctzll(hit) + 1;
    return it0 <= cap ? (int)it0 : -1;
}
__device__ __forceinline__ int warm_chunks(const float* bound, int HV, int64_t it0, int cap, int lane) {
    return warm_from(warm_load(bound, HV, it0, cap, lane), it0, cap, lane);
}

// Whether the segments of this (sequence, head) need the exact start states of the first pass and the merge:
// true when some segment cannot be warm-started within the cap.  The bounds of eight segments are requested
// before the first is looked at (every workgroup of three launches waits for this answer before anything else).
// `warm_of` (optional) receives warm_chunks() of segment `seg`.
__device__ __forceinline__ bool needs_exact_segments(const SegmentPlan& sp, const float* bound, int HV, int lane,
                                                     int seg = -1, int* warm_of = nullptr) {
    bool exact = false;
    for (int j0 = 1; j0 < sp.nseg; j0 += 8) {
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = j0 + e < sp.nseg ? warm_load(bound, HV, (int64_t)(j0 + e) * sp.seg_chunks, sp.warm_cap, lane) : 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (j0 + e >= sp.nseg) break;
            const int wch = warm_from(x[e], (int64_t)(j0 + e) * sp.seg_chunks, sp.warm_cap, lane);
            exact |= wch < 0;
            if (warm_of && j0 + e == seg) *warm_of = wch;
        }
    }
    return exact;
}

// launchers defined next to their kernels
template <typename T> int launch_prepare(const ChunkParams& p, int64_t num_chunks, hipStream_t stream);
// Sequential stage; sp.kind selects whole sequences, pass 1 or pass 2.  Four compute waves and one
// run per workgroup (gdn_chunk_wide.hip) or eight compute waves and two runs (gdn_chunk_pair.hip).
template <typename T> int launch_wide(const ChunkParams& p, SegmentPlan sp, hipStream_t stream);
template <typename T> int launch_pair(const ChunkParams& p, SegmentPlan sp, hipStream_t stream);
int launch_segment_merge(const ChunkParams& p, SegmentPlan sp, hipStream_t stream);
// Sequential stage for 128 < K <= 256 (gdn_chunk_wide256.hip): whole sequences, any V that is a multiple of 8.
template <typename T> int launch_wide256(const ChunkParams& p, hipStream_t stream);

}  // namespace gdn
