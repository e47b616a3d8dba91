// Error reporting shared by all dmlhip_* entry points.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

namespace dml {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return (int)e;
}

}  // namespace dml

extern "C" {
int dmlhip_version(void) { return DMLHIP_VERSION; }
const char* dmlhip_last_error_string(void) { return dml::g_error; }
}
