// Library-wide pieces of the C ABI: version and the thread-local error string.
#include <stdarg.h>
#include <string.h>

#include "common.cuh"

namespace msamp {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return MSAMP_ERR_HIP - static_cast<int>(e);
}

}    // namespace msamp

extern "C" {

int msamp_hip_version(void) { return 100; }

const char* msamp_last_error(void) { return msamp::g_err; }

}    // extern "C"
