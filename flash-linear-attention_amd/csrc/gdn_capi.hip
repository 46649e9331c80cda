// Error channel and version of the C ABI.
#include "gdn_common.h"

namespace gdn {
static thread_local char g_err[512] = {0};
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
}  // namespace gdn

extern "C" int gdn_hip_abi_version(void) { return 4; }
extern "C" const char* gdn_last_error(void) { return gdn::g_err; }
