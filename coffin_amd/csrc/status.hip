// Thread-local error text behind cmi_last_error() and the ABI version.
#include "common.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

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

int compute_units() {
    static std::atomic<int> count[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    int n = count[dev & 63].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
    count[dev & 63].store(n, std::memory_order_relaxed);
    return n;
}

// ------------------------------------------------------------------ options
// Kernel-selection overrides for tests and tuning.  Each is read from its environment variable
// once, when first asked for, and validated there; afterwards only cmi_set_option changes it, so
// the hot path costs one relaxed atomic load per call and never calls getenv.
namespace {
constexpr int UNREAD = INT32_MIN;
std::atomic<int> g_gemm_tile{UNREAD};      // 0 = the library chooses
std::atomic<int> g_gemv_wholerow{UNREAD};  // -1 = the library chooses, 0 = never, 1 = where it can
std::atomic<int> g_w4_decode_waves{0};     // 0 = the library chooses, 4 or 16 wavefronts per workgroup
std::atomic<int> g_w4_decode_chain{0};     // 0 = the library chooses, 1 = never, else a variant code

bool valid_gemm_tile(int v) { return v == 0 || v == 64 || v == 128 || v == 256 || v == 192 || v == 320 || v == 321 || v == 322 || v == 6464 || v == 128192; }
bool valid_wholerow(int v) { return v >= -1 && v <= 1; }

int from_env(const char *name, int fallback, bool (*valid)(int)) {
    const char *e = getenv(name);
    if (!e || !e[0]) return fallback;
    char *end = nullptr;
    const long v = strtol(e, &end, 10);
    if (end == e || *end != '\0' || !valid((int)v)) {
        fprintf(stderr, "coffin_mi355: ignoring %s=%s (not a value this library knows)\n", name, e);
        return fallback;
    }
    return (int)v;
}
}  // namespace

int option_gemm_tile() {
    int v = g_gemm_tile.load(std::memory_order_relaxed);
    if (v == UNREAD) {
        v = from_env("CMI_GEMM_TILE", 0, valid_gemm_tile);
        g_gemm_tile.store(v, std::memory_order_relaxed);
    }
    return v;
}

int option_gemv_wholerow() {
    int v = g_gemv_wholerow.load(std::memory_order_relaxed);
    if (v == UNREAD) {
        v = from_env("CMI_GEMV_WHOLEROW", -1, valid_wholerow);
        g_gemv_wholerow.store(v, std::memory_order_relaxed);
    }
    return v;
}

int option_w4_decode_waves() { return g_w4_decode_waves.load(std::memory_order_relaxed); }
int option_w4_decode_chain() { return g_w4_decode_chain.load(std::memory_order_relaxed); }

}  // namespace cmi

extern "C" int cmi_set_option(const char *name, int value) {
    using namespace cmi;
    CMI_REQUIRE(name, CMI_E_ARG, "cmi_set_option: null name");
    if (!strcmp(name, "gemm_tile")) {
        CMI_REQUIRE(valid_gemm_tile(value), CMI_E_ARG,
                    "cmi_set_option: gemm_tile=%d, expected 0 (library's choice), 64, 128, 192, 256, 320, 321, 322, 6464 or 128192", value);
        g_gemm_tile.store(value, std::memory_order_relaxed);
        return CMI_OK;
    }
    if (!strcmp(name, "gemv_wholerow")) {
        CMI_REQUIRE(valid_wholerow(value), CMI_E_ARG,
                    "cmi_set_option: gemv_wholerow=%d, expected -1 (library's choice), 0 or 1", value);
        g_gemv_wholerow.store(value, std::memory_order_relaxed);
        return CMI_OK;
    }
    if (!strcmp(name, "w4_decode_waves")) {
        CMI_REQUIRE(value == 0 || value == 4 || value == 16, CMI_E_ARG,
                    "cmi_set_option: w4_decode_waves=%d, expected 0 (library's choice), 4 or 16", value);
        g_w4_decode_waves.store(value, std::memory_order_relaxed);
        return CMI_OK;
    }
    if (!strcmp(name, "w4_decode_chain")) {
        const int lanes = value % 100, split = value / 100 % 100, waves = value / 10000;
        CMI_REQUIRE(value == 0 || value == 1 ||
                        ((lanes == 8 || lanes == 16) && (split == 1 || split == 2 || split == 4 || split == 8) &&
                         (waves == 4 || waves == 8 || waves == 16)),
                    CMI_E_ARG,
                    "cmi_set_option: w4_decode_chain=%d, expected 0 (library's choice), 1 (never) or lanes (8, 16) "
                    "+ 100 * wavefronts per row (1, 2, 4, 8) + 10000 * wavefronts per workgroup (4, 8, 16)", value);
        g_w4_decode_chain.store(value, std::memory_order_relaxed);
        return CMI_OK;
    }
    return fail(CMI_E_ARG, "cmi_set_option: unknown option '%s'", name);
}

extern "C" int cmi_abi_version(void) { return 3; }

extern "C" const char *cmi_last_error(void) { return g_error; }
