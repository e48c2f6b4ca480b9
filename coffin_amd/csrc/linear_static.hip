// Quantiser + W4A8 projection for callers that cannot allocate device memory (code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc): the quantised rows and
// their scales go through a fixed array of this library instead of a caller's workspace.
#include "common.hpp"

#include <mutex>

namespace {

using namespace cmi;

constexpr size_t ALIGN = 256;
constexpr size_t round_up(size_t v) { return (v + ALIGN - 1) / ALIGN * ALIGN; }

// Fixed workspace of the entry point that allocates nothing: 8 MiB of quantised rows and
// scales for up to 16384 rows.  Every GPU the library runs on holds its own copy until the
// process ends.
constexpr size_t STATIC_XQ_BYTES = 8u << 20;
constexpr int STATIC_MAX_ROWS = 16384;
constexpr size_t STATIC_BYTES = STATIC_XQ_BYTES + round_up(sizeof(float) * STATIC_MAX_ROWS);
static __device__ __align__(256) unsigned char scratch[STATIC_BYTES];

// Device address of `scratch` on the current device.  The array's name is only a host-side
// handle: the address each GPU holds its copy at is asked for once per device, with that
// device current, and kept.
constexpr int MAX_DEVICES = 64;
unsigned char *g_scratch_ptr[MAX_DEVICES];
std::mutex g_scratch_lock;

int static_workspace(unsigned char **out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(CMI_E_HIP, "cmi_linear_w4a8_bf16_static: no current device");
    CMI_REQUIRE(dev >= 0 && dev < MAX_DEVICES, CMI_E_UNSUPPORTED,
                "cmi_linear_w4a8_bf16_static: device ordinal %d above %d", dev, MAX_DEVICES - 1);
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        const hipError_t err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !p)
            return fail(CMI_E_HIP, "cmi_linear_w4a8_bf16_static: hipGetSymbolAddress: %s", hipGetErrorString(err));
        g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
    }
    *out = g_scratch_ptr[dev];
    return CMI_OK;
}

}  // namespace

extern "C" int cmi_linear_w4a8_bf16_static(const uint8_t *w4, const float *ws, const void *x, void *y, int M, int N,
                                           int K, int gs, void *stream) {
    CMI_REQUIRE(M >= 0 && N >= 1 && K >= 1, CMI_E_ARG, "cmi_linear_w4a8_bf16_static: bad shape M=%d N=%d K=%d", M,
                N, K);
    if (M == 0) return CMI_OK;
    CMI_REQUIRE(w4 && ws && x && y, CMI_E_ARG, "cmi_linear_w4a8_bf16_static: null pointer");
    const int Kd = cmi_w4_device_k(K, gs);
    CMI_REQUIRE(Kd > 0, CMI_E_UNSUPPORTED, "cmi_linear_w4a8_bf16_static: group size %d, the kernels are built for 64, 128 and 256", gs);
    CMI_REQUIRE(M <= STATIC_MAX_ROWS && (size_t)M * Kd <= STATIC_XQ_BYTES, CMI_E_UNSUPPORTED,
                "cmi_linear_w4a8_bf16_static: M=%d x K=%d exceeds the fixed workspace (M <= %d, M*K <= %zu); "
                "use cmi_linear_w4a8_bf16 with a workspace of cmi_linear_workspace_bytes(M, K)",
                M, K, STATIC_MAX_ROWS, STATIC_XQ_BYTES);
    unsigned char *base = nullptr;
    if (const int rc = static_workspace(&base)) return rc;
    int8_t *xq = reinterpret_cast<int8_t *>(base);
    float *xs = reinterpret_cast<float *>(base + STATIC_XQ_BYTES);
    return linear_w4a8_rows(w4, ws, x, y, M, N, K, gs, xq, xs, stream);
}
