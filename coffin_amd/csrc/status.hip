// Thread-local error text behind cmi_last_error() and the ABI version.
#include "common.hpp"

#include <cstdarg>
#include <cstdio>

namespace {
thread_local char g_error[512] = "";
}

namespace cmi {

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what) {
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(CMI_E_HIP, "%s: %s", what, hipGetErrorString(err));
    return CMI_OK;
}

int reserve_lds(const void *kernel, int bytes, std::atomic<uint64_t> &devices, const char *who) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(CMI_E_HIP, "%s: no current device", who);
    const uint64_t bit = 1ull << (dev & 63);
    if (devices.load(std::memory_order_acquire) & bit) return CMI_OK;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
        return fail(CMI_E_HIP, "%s: cannot reserve %d bytes of LDS", who, bytes);
    devices.fetch_or(bit, std::memory_order_release);
    return CMI_OK;
}

}  // namespace cmi

extern "C" int cmi_abi_version(void) { return 1; }

extern "C" const char *cmi_last_error(void) { return g_error; }
