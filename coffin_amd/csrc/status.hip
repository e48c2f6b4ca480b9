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

}  // namespace cmi

extern "C" int cmi_abi_version(void) { return 1; }

extern "C" const char *cmi_last_error(void) { return g_error; }
