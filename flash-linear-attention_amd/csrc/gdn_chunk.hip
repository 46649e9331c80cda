// C entry points of the chunked prefill (64-token chunks; head dims that are multiples of 8, K <= 256): argument
// checks, workspace layout and the choice of kernels.  The kernels live in gdn_chunk_prepare.hip (chunk-parallel
// stage) and gdn_chunk_wide.hip, gdn_chunk_pair.hip, gdn_chunk_wide256.hip (sequential stage).
#include "gdn_chunk_common.h"

namespace gdn {

constexpr int STAGE_PREPARE = 1, STAGE_SCAN = 2;

template <typename T>
static int launch_chunk(const ChunkParams& p0, int64_t num_chunks, int stages, hipStream_t stream) {
    ChunkParams p = p0;
    // One workgroup per (sequence, head) walks the chunks of the sequence, or time is cut into
    // segments (plan_segments).  Either way a workgroup can also carry two runs that read the same k rows (two value heads of
    // a q/k head; in pass 1 the S and M runs of one head).  That halves the number of workgroups and
    // runs a pair about 1.25 times as fast as two single runs one after the other, so it pays as soon
    // as the single runs would not all fit on the chip at once.
    if (p.K > 128) {
        // wide keys: whole sequences, a workgroup per 64 value columns; the scan forms P itself
        p.want_P = (p.flags & GDN_FLAG_RECORD_P) != 0;
        if (stages & STAGE_PREPARE) {
            if (int rc = launch_prepare<T>(p, num_chunks, stream)) return rc;
        }
        return (stages & STAGE_SCAN) ? launch_wide256<T>(p, stream) : GDN_OK;
    }
    const int64_t G = p.HV / p.H;
    const int nseg = plan_segments(p.N, p.HV, p.NT, num_chunks, p.cu_seqlens == nullptr, p.flags);
    const bool segments = nseg > 0;
    // (head dims up to 64 have a one-run kernel with a quarter-size state; the two-run kernel would do the full 128 x 128 work)
    const bool small = p.K <= 64 && p.V <= 64;
    const bool no_pair = (p.flags & GDN_FLAG_SCAN_NO_PAIR) || small, force_pair = (p.flags & GDN_FLAG_SCAN_PAIR) && !small;
    // (full runs in pairs: an even number of value heads per q/k head, and all 128 value columns real: the two-run
    // kernel counts its output stores, which every wave must therefore have)
    const bool pair_full_ok = G % 2 == 0 && p.V == 128;
    auto use_pair = [&](bool possible, int64_t single_workgroups) {
        return possible && !no_pair && (force_pair || single_workgroups > 256);
    };
    const bool pass2_pairs = segments && use_pair(pair_full_ok, p.NH * nseg);
    const bool whole_pairs = !segments && use_pair(pair_full_ok, p.NH);
    p.want_P = (p.flags & GDN_FLAG_RECORD_P) != 0;       // every scan kernel forms P itself
    if (stages & STAGE_PREPARE) {
        int rc = launch_prepare<T>(p, num_chunks, stream);
        if (rc) return rc;
    }
    if (!(stages & STAGE_SCAN)) return GDN_OK;
    SegmentPlan sp = {};
    if (!segments) {
        sp.kind = WIDE_WHOLE;
        return whole_pairs ? launch_pair<T>(p, sp, stream) : launch_wide<T>(p, sp, stream);
    }
    sp.nseg = nseg;
    sp.seg_chunks = (int)((p.NT + nseg - 1) / nseg);
    const size_t slots = (size_t)p.NH * nseg;
    sp.sloc = p.ws.Seg;
    sp.mseg = p.ws.Seg + slots * 16384;
    sp.sin = p.ws.Seg + 2 * slots * 16384;
    // Segments start warm where the decay allows it (see WARM_LOG2); the first pass and the merge then only serve
    // the heads that need exact start states, and their workgroups for the other heads return at once.  Not with two
    // runs per workgroup in pass 2: the two heads would want different starts.
    if (!(p.flags & GDN_FLAG_SCAN_NO_WARM) && !pass2_pairs) {
        sp.bound = p.ws.Bound;
        // a warm-up of w chunks costs w more steps; the exact start costs about 1.2 steps per chunk of the segment
        // (first pass) plus the merge
        sp.warm_cap = std::min(WARM_CAP_MAX, sp.seg_chunks + sp.seg_chunks / 4 + 6);
    }
    int rc;
    sp.kind = WIDE_PASS1;
    if ((rc = use_pair(true, 2 * p.NH * (nseg - 1)) ? launch_pair<T>(p, sp, stream) : launch_wide<T>(p, sp, stream))) return rc;
    if ((rc = launch_segment_merge(p, sp, stream))) return rc;
    sp.kind = WIDE_PASS2;
    return pass2_pairs ? launch_pair<T>(p, sp, stream) : launch_wide<T>(p, sp, stream);
}

}  // namespace gdn

// K, V multiples of 8: both up to 128, or wide keys (128 < K <= 256) with any number of value columns
static bool chunk_dims_ok(int64_t K, int64_t V) {
    return K >= 8 && V >= 8 && K % 8 == 0 && V % 8 == 0 && (K <= 128 ? V <= 128 : (K <= 256 && V <= 8192));
}

// bytes of workspace for the plan that launch_chunk will choose
static size_t chunk_workspace_need(int64_t N, int64_t T, int64_t num_chunks, int64_t H, int64_t HV, int64_t K, int64_t V, bool packed,
                                   uint32_t flags, char* base, gdn::ChunkWs* ws) {
    using namespace gdn;
    if (K > 128) {                      // wide keys: segment matrices of their own size, none for whole sequences
        const int nseg = plan_segments256(N, H, HV, V, (T + CH - 1) / CH, !packed, flags);
        return ws_layout(num_chunks, HV, nseg > 1 ? (int64_t)nseg * N * HV : 0, base, ws, seg256_floats(V));
    }
    const int nseg = plan_segments(N, HV, (T + CH - 1) / CH, num_chunks, !packed, flags);
    return ws_layout(num_chunks, HV, (int64_t)nseg * N * HV, base, ws);
}

extern "C" size_t gdn_chunk_workspace_bytes(int64_t N, int64_t T, int64_t num_chunks, int64_t H, int64_t HV, int64_t K, int64_t V,
                                            int packed, uint32_t flags) {
    if (!chunk_dims_ok(K, V) || num_chunks < 0 || N < 1 || T < 0 || H < 1 || HV < 1) return 0;
    return chunk_workspace_need(N, T, num_chunks, H, HV, K, V, packed != 0, flags, nullptr, nullptr);
}

static int chunk_entry(
    const char* who, int stages,
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    void* workspace, size_t workspace_bytes,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    using namespace gdn;
    GDN_CHECK_ARG(T == 0 || (q && k && v && beta && o), GDN_ERR_INVALID, "%s: q, k, v, beta, o must not be NULL", who);
    GDN_CHECK_ARG(g || !A_log, GDN_ERR_INVALID, "%s: A_log given without g", who);
    GDN_CHECK_ARG(B >= 1 && T >= 0 && H >= 1 && HV >= 1 && N >= 1, GDN_ERR_INVALID, "%s: non-positive dimension", who);
    GDN_CHECK_ARG(!dt_bias || A_log, GDN_ERR_INVALID, "%s: dt_bias without A_log", who);
    GDN_CHECK_ARG(!(flags & GDN_FLAG_NEG_EIGVAL) || (flags & GDN_FLAG_BETA_SIGMOID), GDN_ERR_INVALID, "%s: GDN_FLAG_NEG_EIGVAL needs GDN_FLAG_BETA_SIGMOID", who);
    GDN_CHECK_ARG(!(flags & GDN_FLAG_SCAN_NO_PAIR) || !(flags & GDN_FLAG_SCAN_PAIR), GDN_ERR_INVALID, "%s: GDN_FLAG_SCAN_PAIR and GDN_FLAG_SCAN_NO_PAIR exclude each other", who);
    GDN_CHECK_ARG(HV % H == 0, GDN_ERR_INVALID, "%s: HV=%lld not divisible by H=%lld", who, (long long)HV, (long long)H);
    GDN_CHECK_ARG(chunk_dims_ok(K, V), GDN_ERR_UNSUPPORTED,
                  "%s: head dims must be multiples of 8, K, V <= 128 or 128 < K <= 256 (got K=%lld V=%lld)", who, (long long)K, (long long)V);
    GDN_CHECK_ARG(qkv_dtype == GDN_DTYPE_BF16 || qkv_dtype == GDN_DTYPE_F16, GDN_ERR_UNSUPPORTED,
                  "%s: q/k/v must be bf16 or f16", who);
    GDN_CHECK_ARG(HV <= 65535 && num_chunks * H < (1ll << 31), GDN_ERR_UNSUPPORTED, "%s: too many heads or chunks for one launch", who);
    if (cu_seqlens) {
        GDN_CHECK_ARG(B == 1, GDN_ERR_INVALID, "%s: with cu_seqlens B must be 1", who);
        GDN_CHECK_ARG((chunk_table || num_chunks == 0) && chunk_offsets, GDN_ERR_INVALID, "%s: packed input needs chunk_table and chunk_offsets", who);
    } else {
        GDN_CHECK_ARG(N == B, GDN_ERR_INVALID, "%s: without cu_seqlens N must equal B", who);
        GDN_CHECK_ARG(num_chunks == B * ((T + CH - 1) / CH), GDN_ERR_INVALID, "%s: num_chunks does not match B and T", who);
    }
    GDN_CHECK_ARG(((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0 && ((uintptr_t)h0 % 16) == 0 &&
                      ((uintptr_t)ht % 16) == 0 && ((uintptr_t)workspace % 256) == 0,
                  GDN_ERR_INVALID, "%s: q/k/v/h0/ht must be 16-byte and the workspace 256-byte aligned", who);
    hipStream_t s = (hipStream_t)stream;
    if (T == 0 || num_chunks == 0) {
        // no token anywhere: the final states are the initial ones
        if (ht && (stages & gdn::STAGE_SCAN)) return launch_state_copy(h0, ht, N * HV * K * V, s);
        return GDN_OK;
    }
    ChunkParams p;
    const size_t need = chunk_workspace_need(N, T, num_chunks, H, HV, K, V, cu_seqlens != nullptr, flags, (char*)workspace, &p.ws);
    GDN_CHECK_ARG(workspace && workspace_bytes >= need, GDN_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who,
                  need, workspace_bytes);
    p.q = q; p.k = k; p.v = v; p.g = g; p.beta = beta; p.A_log = A_log; p.dt_bias = dt_bias; p.h0 = h0; p.ht = ht; p.o = o;
    p.cu_seqlens = cu_seqlens; p.chunk_table = chunk_table; p.chunk_offsets = chunk_offsets;
    p.T = T; p.H = (int)H; p.HV = (int)HV; p.N = N; p.NT = (T + CH - 1) / CH; p.K = (int)K; p.V = (int)V;
    p.scale = scale; p.gb_dtype = gb_dtype; p.flags = flags & ~FLAG_Q_NORM_IN_SCAN; p.NH = N * HV;
    if (q_norm_in_scan(flags, K, V, num_chunks * HV)) p.flags |= FLAG_Q_NORM_IN_SCAN;
    return qkv_dtype == GDN_DTYPE_BF16 ? launch_chunk<bf16_t>(p, num_chunks, stages, s)
                                       : launch_chunk<f16_t>(p, num_chunks, stages, s);
}

#define GDN_CHUNK_ARGS                                                                          \
    const void *q, const void *k, const void *v, const void *g, const void *beta,               \
    const float *A_log, const float *dt_bias,                                                   \
    const float *h0, float *ht, void *o,                                                        \
    const void *cu_seqlens, const void *chunk_table, const void *chunk_offsets,                 \
    void *workspace, size_t workspace_bytes,                                                    \
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,                          \
    int64_t N, int64_t num_chunks,                                                              \
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void *stream
#define GDN_CHUNK_PASS                                                                          \
    q, k, v, g, beta, A_log, dt_bias, h0, ht, o, cu_seqlens, chunk_table, chunk_offsets, workspace, workspace_bytes, \
    B, T, H, HV, K, V, N, num_chunks, scale, qkv_dtype, gb_dtype, flags, stream

extern "C" int gdn_chunk_fwd(GDN_CHUNK_ARGS) {
    return chunk_entry("gdn_chunk_fwd", gdn::STAGE_PREPARE | gdn::STAGE_SCAN, GDN_CHUNK_PASS);
}
extern "C" int gdn_chunk_fwd_prepare(GDN_CHUNK_ARGS) {
    return chunk_entry("gdn_chunk_fwd_prepare", gdn::STAGE_PREPARE, GDN_CHUNK_PASS);
}
extern "C" int gdn_chunk_fwd_scan(GDN_CHUNK_ARGS) {
    return chunk_entry("gdn_chunk_fwd_scan", gdn::STAGE_SCAN, GDN_CHUNK_PASS);
}

// ---------------------------------------------------------------------------------------------
// gdn_chunk_fwd without any allocation: the workspace is a fixed array in device memory that
// belongs to the library (one copy per GPU, held until the process ends).
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[GDN_CHUNK_STATIC_WORKSPACE_BYTES];

// Device address of `scratch` on the current device.  The array's name is only a handle on the host:
// its address on each GPU comes from hipGetSymbolAddress, asked once per device with that device current.
static int static_workspace(const char* who, void** out) {
    static void* addr[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return gdn::check_launch(who);
    GDN_CHECK_ARG(dev >= 0 && dev < 64, GDN_ERR_UNSUPPORTED, "%s: device index %d not supported", who, dev);
    void* p = __atomic_load_n(&addr[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            gdn::set_error("%s: hipGetSymbolAddress(scratch): %s", who, hipGetErrorString(e));
            (void)hipGetLastError();
            return GDN_ERR_LAUNCH;
        }
        __atomic_store_n(&addr[dev], p, __ATOMIC_RELEASE);      // (every thread that asks gets the same address)
    }
    *out = p;
    return GDN_OK;
}

extern "C" int gdn_chunk_fwd_static(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    const float* A_log, const float* dt_bias,
    const float* h0, float* ht, void* o,
    const void* cu_seqlens, const void* chunk_table, const void* chunk_offsets,
    int64_t B, int64_t T, int64_t H, int64_t HV, int64_t K, int64_t V,
    int64_t N, int64_t num_chunks,
    float scale, int qkv_dtype, int gb_dtype, uint32_t flags, void* stream) {
    const char* who = "gdn_chunk_fwd_static";
    GDN_CHECK_ARG(chunk_dims_ok(K, V) && N >= 1 && T >= 0 && HV >= 1 && num_chunks >= 0, GDN_ERR_INVALID,
                  "%s: bad dimensions", who);
    // The plan with time segments needs room for their matrices; when only that does not fit, whole sequences do.
    size_t need = chunk_workspace_need(N, T, num_chunks, H, HV, K, V, cu_seqlens != nullptr, flags, nullptr, nullptr);
    if (need > GDN_CHUNK_STATIC_WORKSPACE_BYTES && !(flags & GDN_FLAG_SCAN_SEGMENTS)) {
        flags |= GDN_FLAG_SCAN_WIDE;
        need = chunk_workspace_need(N, T, num_chunks, H, HV, K, V, cu_seqlens != nullptr, flags, nullptr, nullptr);
    }
    GDN_CHECK_ARG(need <= GDN_CHUNK_STATIC_WORKSPACE_BYTES, GDN_ERR_WORKSPACE,
                  "%s: this input needs %zu bytes of workspace, the built-in one holds %zu (%lld records of one chunk and "
                  "value head); use gdn_chunk_fwd with a workspace of the caller",
                  who, need, (size_t)GDN_CHUNK_STATIC_WORKSPACE_BYTES,
                  (long long)(GDN_CHUNK_STATIC_WORKSPACE_BYTES / gdn::REC_BYTES));
    void* workspace = nullptr;
    if (int rc = static_workspace(who, &workspace)) return rc;
    const size_t workspace_bytes = GDN_CHUNK_STATIC_WORKSPACE_BYTES;
    return chunk_entry(who, gdn::STAGE_PREPARE | gdn::STAGE_SCAN, GDN_CHUNK_PASS);
}
