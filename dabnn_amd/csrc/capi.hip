// Error reporting and device queries behind the C ABI.
#include <stdarg.h>

#include "common.h"

namespace dab {

std::string &last_error() {
    static thread_local std::string msg;
    return msg;
}

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

int simd_count() {
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 1024;
    if (cached[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cached[dev] = cus * 4;
    }
    return cached[dev];
}

}  // namespace dab

extern "C" const char *dab_last_error(void) { return dab::last_error().c_str(); }

extern "C" int dab_version(void) { return 1; }

extern "C" int dab_device_info(int *cu_count, int *clock_khz) {
    using namespace dab;
    int dev = 0;
    DAB_HIP(hipGetDevice(&dev));
    if (cu_count) DAB_HIP(hipDeviceGetAttribute(cu_count, hipDeviceAttributeMultiprocessorCount, dev));
    if (clock_khz) DAB_HIP(hipDeviceGetAttribute(clock_khz, hipDeviceAttributeClockRate, dev));
    return DAB_OK;
}
