// Host-side pieces shared by every entry point: the per-thread error string and launch checking.
#include <stdarg.h>
#include <stdio.h>

#include "svdq_common.h"

namespace svdq {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: HIP launch failed: %s", what, hipGetErrorString(e));
        return SVDQ_E_LAUNCH;
    }
    return SVDQ_OK;
}

}  // namespace svdq

extern "C" const char *svdq_last_error(void) { return svdq::g_err; }
extern "C" int svdq_abi_version(void) { return SVDQ_ABI_VERSION; }
