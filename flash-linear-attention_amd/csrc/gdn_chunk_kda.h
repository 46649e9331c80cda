// Types shared by the chunked KDA forward (gdn_chunk_kda.hip) and the backward that runs its chunk-parallel kernel again
// (gdn_chunk_bwd.hip).
#pragma once
#include "gdn_tiles.h"

namespace gdn {

constexpr int PG = BD + 4;           // pitch of the fp32 gate tile

// Am, Gk: for the backward pass (NULL otherwise): A = (I + diag(beta) M)^-1 [64][64] in the operand type and the
// running sums of the log decays [64][128] fp32, per unit
struct KdaWs { void* Wm; void* Um; void* QG; void* KG; void* Pm; float* EGL; void* Am; float* Gk; };
inline size_t kda_ws_layout(int64_t units, char* base, KdaWs* ws) {
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += ws_align(bytes); return base ? (void*)(base + o) : nullptr; };
    const size_t u = (size_t)units;
    void* Wm = take(u * 64 * BD * 2); void* Um = take(u * 64 * BD * 2);
    void* QG = take(u * 64 * BD * 2); void* KG = take(u * 64 * BD * 2);
    void* Pm = take(u * 64 * 64 * 2); void* EGL = take(u * BD * 4);
    if (ws) *ws = KdaWs{Wm, Um, QG, KG, Pm, (float*)EGL, nullptr, nullptr};
    return off;
}

struct KdaParams {
    const void* q; const void* k; const void* v; const float* g; const void* beta;
    const void* pk; const void* gs;                                             // comba: the second key, the log decay per token and head
    const float* A_log; const float* gk_bias; float gk_lower; int gk_act;      // gate activation, as in the token recurrence
    const float* h0; float* ht; void* o;
    void* hs;                           // the state in front of every chunk [num_chunks][HV][128][128] in the operand type, or NULL
    const void* cu_seqlens; const void* chunk_table; const void* chunk_offsets;
    KdaWs ws;
    int64_t T; int H, HV; int64_t N; int64_t NT;
    float scale; int gb_dtype; uint32_t flags;
};

// the chunk-parallel kernel of the forward on its own: writes w, u, qg, kg, P, e^Gam_last and, where the pointers are set, A and Gam
int launch_kda_prepare(const KdaParams& p, int64_t num_chunks, int qkv_dtype, hipStream_t stream);

}  // namespace gdn
