// Error reporting and device facts for the C ABI.
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "mynn_common.h"

namespace mynn {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}
int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}
LaunchTimer &launch_timer() {
    static thread_local LaunchTimer t;
    return t;
}

int hip_fail(hipError_t e, const char *what) {
    snprintf(g_err, sizeof g_err, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
    return (int)e;
}

}  // namespace mynn

extern "C" const char *mynn_last_error(void) { return mynn::g_err; }
extern "C" int mynn_version(void) { return 1; }

extern "C" int mynn_device_info(int *cu_count, int *wave_size, int *lds_bytes, char *arch, size_t arch_len) {
    int dev = 0;
    MYNN_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    MYNN_HIP(hipGetDeviceProperties(&prop, dev));
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (wave_size) *wave_size = prop.warpSize;
    if (lds_bytes) *lds_bytes = (int)prop.sharedMemPerBlock;
    if (arch && arch_len) {
        strncpy(arch, prop.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    return 0;
}
