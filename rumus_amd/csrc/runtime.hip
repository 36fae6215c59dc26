// Runtime entry points: status reporting, device selection, stream sync.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "common.h"

namespace rumus {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return RUMUS_HIP_OK;
    return set_error(RUMUS_HIP_EHIP, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace rumus

extern "C" {

int rumus_hip_init(int device) {
    int count = 0;
    if (int rc = rumus::check_hip(hipGetDeviceCount(&count), "hipGetDeviceCount")) return rc;
    RUMUS_REQUIRE(device >= 0 && device < count, "rumus_hip_init: device %d of %d", device, count);
    if (int rc = rumus::check_hip(hipSetDevice(device), "hipSetDevice")) return rc;
    hipDeviceProp_t prop;
    if (int rc = rumus::check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties"))
        return rc;
    // The kernels are built for gfx950 only; refuse anything else up front
    // instead of failing at the first launch.
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return rumus::set_error(RUMUS_HIP_EINVAL, "rumus_hip_init: device is %s, library is gfx950 only",
                                prop.gcnArchName);
    return RUMUS_HIP_OK;
}

const char* rumus_hip_last_error(void) { return rumus::g_err; }

const char* rumus_hip_version(void) { return "rumus-hip 0.1.0 gfx950"; }

int rumus_hip_sync(rumus_hip_stream_t stream) {
    return rumus::check_hip(hipStreamSynchronize(rumus::as_stream(stream)), "hipStreamSynchronize");
}

}  // extern "C"
