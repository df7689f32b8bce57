// Error reporting and version entry points of the C ABI.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

namespace odl {

static thread_local char g_err[512] = "";

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return ODL_OK;
    return set_error(ODL_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace odl

extern "C" int odl_fp8_abi_version(void) { return 6; }

extern "C" const char *odl_fp8_last_error(void) { return odl::g_err; }
