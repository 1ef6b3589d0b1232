// Library identity, per-thread error channel and device query.
#include "common.h"

#include <string.h>

namespace mi355x {

static thread_local char g_last_error[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* kernel_name) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return set_error(MI355X_ERR_LAUNCH, "%s: launch failed: %s", kernel_name, hipGetErrorString(e));
    return MI355X_OK;
}

}  // namespace mi355x

extern "C" {

int mi355x_version(void) { return MI355X_ONNX_VERSION; }

const char* mi355x_last_error(void) { return mi355x::g_last_error; }

int mi355x_device_cu_count(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return cus;
}

}  // extern "C"
