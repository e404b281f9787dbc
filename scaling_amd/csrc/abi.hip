// Status / error plumbing and device check of libmi355_layer.so.
#include "common.h"
#include <string.h>

static thread_local char g_err[512] = "";

void mi_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int mi_fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int mi_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mi_fail(MI_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MI_OK;
}

extern "C" {

int mi_version(void) { return MI355_LAYER_VERSION; }

const char* mi_last_error(void) { return g_err; }

const char* mi_status_string(int status) {
    switch (status) {
        case MI_OK: return "MI_OK";
        case MI_E_NULL: return "MI_E_NULL";
        case MI_E_DTYPE: return "MI_E_DTYPE";
        case MI_E_SHAPE: return "MI_E_SHAPE";
        case MI_E_ALIGN: return "MI_E_ALIGN";
        case MI_E_WORKSPACE: return "MI_E_WORKSPACE";
        case MI_E_LAUNCH: return "MI_E_LAUNCH";
        case MI_E_ARCH: return "MI_E_ARCH";
        default: return "MI_E_UNKNOWN";
    }
}

int mi_check_device(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return mi_fail(MI_E_ARCH, "no HIP device available");
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        return mi_fail(MI_E_ARCH, "hipGetDeviceProperties failed");
    }
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return mi_fail(MI_E_ARCH, "device %d is %s, this library is built for gfx950 only", dev, prop.gcnArchName);
    return MI_OK;
}

}  // extern "C"
