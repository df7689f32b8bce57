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

// Compute units of the device that is current on the calling thread.  One slot per device ordinal: a
// process that drives several GPUs sizes every grid for the GPU it launches on.  The slots are plain
// ints: two threads that fill one at the same time write the same value.
int device_cu_count() {
    constexpr int kMaxDevices = 64;
    static int cached[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
    int cus = cached[dev];
    if (cus == 0) {
        hipDeviceProp_t prop;
        cus = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        cached[dev] = cus;
    }
    return cus;
}

}  // namespace odl

extern "C" int odl_fp8_abi_version(void) { return 16; }

extern "C" int odl_fp8_init_device(void) {
    if (!odl::scratch_for_current_device("odl_fp8_init_device")) return ODL_ERR_LAUNCH;
    if (!odl::unit_scale_for_current_device("odl_fp8_init_device")) return ODL_ERR_LAUNCH;
    (void)odl::device_cu_count();
    return ODL_OK;
}

extern "C" const char *odl_fp8_last_error(void) { return odl::g_err; }
