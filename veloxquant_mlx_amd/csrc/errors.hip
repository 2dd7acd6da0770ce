// Thread-local error text and the small introspection entry points.
#include <stdarg.h>
#include <string.h>

#include "common.hpp"

namespace vq {

static thread_local char g_err[512] = {0};

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace vq

extern "C" int vq_abi_version(void) { return 16; }

extern "C" int vq_last_error(char *buf, size_t n) {
    size_t len = strlen(vq::g_err);
    if (buf && n) {
        size_t c = len < n - 1 ? len : n - 1;
        memcpy(buf, vq::g_err, c);
        buf[c] = 0;
    }
    return (int)len;
}

extern "C" int vq_device_count(void) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return vq::fail(VQ_ERR_HIP, "hipGetDeviceCount: %s", hipGetErrorString(e));
    return n;
}
