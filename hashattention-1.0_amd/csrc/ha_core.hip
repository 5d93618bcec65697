// Library-wide host plumbing: version, status strings, thread-local error text, device probe.
#include <stdarg.h>
#include <string.h>

#include "ha_common.h"

static thread_local char g_err[512] = "";

void ha_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int ha_require_device(void) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();  // clear the sticky "no device" error
        HA_FAIL(HA_ERR_NO_DEVICE, "no HIP device visible (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    }
    return HA_OK;
}

extern "C" {

int ha_version(void) { return HA_VERSION; }

const char *ha_status_string(int status) {
    switch (status) {
        case HA_OK: return "ok";
        case HA_ERR_NULL_POINTER: return "null pointer";
        case HA_ERR_BAD_SHAPE: return "unsupported shape or size";
        case HA_ERR_BAD_DTYPE: return "unsupported dtype";
        case HA_ERR_MISALIGNED: return "misaligned pointer or stride";
        case HA_ERR_WORKSPACE: return "workspace missing or too small";
        case HA_ERR_NO_DEVICE: return "no HIP device";
        case HA_ERR_HIP: return "HIP runtime error";
        default: return "unknown status";
    }
}

const char *ha_last_error_string(void) { return g_err; }

int ha_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

}  // extern "C"
