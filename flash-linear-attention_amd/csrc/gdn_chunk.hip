// placeholder until the chunk kernels land
#include "gdn_common.h"
extern "C" size_t gdn_chunk_workspace_bytes(int64_t, int64_t, int64_t, int64_t, int64_t) { return 0; }
extern "C" int gdn_chunk_fwd(
    const void*, const void*, const void*, const void*, const void*,
    const float*, float*, void*, const void*, const void*, const void*,
    void*, size_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
    float, int, int, uint32_t, void*) {
    gdn::set_error("gdn_chunk_fwd: not built");
    return GDN_ERR_UNSUPPORTED;
}
