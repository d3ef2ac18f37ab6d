// Error reporting and version of the C ABI.
#include "akv_common.h"

#include <stdarg.h>

namespace akv {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return AKV_ERR_LAUNCH;
    }
    return AKV_OK;
}

}  // namespace akv

extern "C" int akv_version(void) { return 100; }

extern "C" const char *akv_last_error(void) { return akv::g_error; }
