// Error reporting and version for libflashnn_hip.so.
#include "fnn_common.h"

#include <stdarg.h>
#include <stdio.h>

namespace fnn {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: HIP launch failed: %s", what, hipGetErrorString(e));
        return FNN_ERR_HIP;
    }
    return FNN_OK;
}

}  // namespace fnn

extern "C" int fnn_version(void) { return 1; }
extern "C" const char* fnn_last_error(void) { return fnn::g_err; }
