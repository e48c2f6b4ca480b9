// Whole projections from bf16 activations for the integer paths: per-token quantiser + W8A8
// GEMM, and quantiser + W4A8 GEMV / GEMM (or the GEMV with the quantiser folded in where that
// is the faster route).  One call per projection instead of two keeps the host side of a decode
// step short, and puts the choice of route next to the kernels it chooses between.
//
// The quantised rows (xq int8 [M,K]) and their scales (xs fp32 [M]) live in a workspace that the
// caller brings.
#include "common.hpp"

namespace {

using namespace cmi;

constexpr size_t ALIGN = 256;
constexpr size_t round_up(size_t v) { return (v + ALIGN - 1) / ALIGN * ALIGN; }

// Whether `rows` bf16 rows go through the W4A8 GEMV that quantises them itself (one launch).
// That kernel lets every workgroup redo the quantisation.  One row of K <= 5120 always (5120 ->
// 25600: 15.2 us against 2.3 + 13.0 us as two launches, 5120 -> 9728: 8.2 against 2.3 + 6.9); longer
// rows lose where many workgroups each quantise them (K > 5120 with N >= 8192), and win for up to
// two rows elsewhere; beyond K = 10240 only the two-launch route has a fast kernel.
bool w4_fused_route(int rows, int N, int K) {
    if (K <= 5120) return rows <= 1;
    if (N >= 8192 || K > 10240) return false;
    return rows <= 2;
}

}  // namespace

int cmi::linear_w4a8_rows(const uint8_t *w4, const float *ws, const void *x, void *y, int M, int N, int K,
                          int gs, int8_t *xq, float *xs, void *stream) {
    // the device copy of the weight has rows of Kd >= K codes (whole groups, whole 128-element
    // steps, cmi_w4_device_k); the quantised rows are padded with zeros to match
    const int Kd = cmi_w4_device_k(K, gs);
    CMI_REQUIRE(Kd > 0, CMI_E_UNSUPPORTED, "cmi_linear_w4a8_bf16: group size %d, the kernels are built for 64, 128 and 256", gs);
    if (gs == 128 && Kd == K && w4_fused_route(M, N, K)) {
        const int rc = cmi_gemv_w4a8_bf16(w4, ws, x, y, nullptr, nullptr, nullptr, M, N, K, gs, stream);
        if (rc != CMI_E_UNSUPPORTED) return rc;
    }
    if (const int rc = quant_act_i8_padded(x, xq, xs, M, K, Kd, stream)) return rc;
    // up to 16 rows the GEMV entry; beyond, the GEMM entry (which itself goes through the
    // read-once kernels while they are cheaper than the tile pipeline)
    if (M <= 16) return cmi_gemv_w4a8(w4, ws, xq, xs, y, nullptr, M, N, Kd, gs, stream);
    return cmi_gemm_w4a8(w4, ws, xq, xs, y, nullptr, M, N, Kd, gs, stream);
}

namespace {

int split_workspace(const char *who, void *workspace, size_t bytes, int M, int K, int8_t **xq, float **xs) {
    CMI_REQUIRE(workspace, CMI_E_ARG, "%s: null workspace", who);
    CMI_REQUIRE(aligned(workspace, 16), CMI_E_ARG, "%s: workspace must be 16-byte aligned", who);
    const size_t need = cmi_linear_workspace_bytes(M, K);
    CMI_REQUIRE(bytes >= need, CMI_E_ARG, "%s: workspace of %zu bytes, %zu needed for M=%d K=%d", who, bytes, need, M, K);
    *xq = static_cast<int8_t *>(workspace);
    *xs = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + round_up((size_t)M * K));
    return CMI_OK;
}

}  // namespace

extern "C" size_t cmi_linear_workspace_bytes(int M, int K) {
    if (M <= 0 || K <= 0) return 0;
    return round_up((size_t)M * K) + round_up(sizeof(float) * (size_t)M);
}

constexpr int ARRIVALS = 256;  // split-K arrival counters behind xq and xs

extern "C" size_t cmi_linear_w8a8_workspace_bytes(int M, int N, int K) {
    const size_t base = cmi_linear_workspace_bytes(M, K);
    if (base == 0 || N <= 0) return base;
    const size_t split = gemm_w8a8_split_bytes(M, N, K);
    return split ? base + round_up(sizeof(int) * ARRIVALS) + split : base;
}

extern "C" int cmi_linear_w8a8_bf16(const void *x, const int8_t *wq, const float *ws, void *y, int M, int N, int K,
                                    int ldy, void *workspace, size_t workspace_bytes, void *stream) {
    CMI_REQUIRE(M >= 0 && N >= 1 && K >= 16, CMI_E_ARG, "cmi_linear_w8a8_bf16: bad shape M=%d N=%d K=%d", M, N, K);
    if (M == 0) return CMI_OK;
    CMI_REQUIRE(x && wq && ws && y, CMI_E_ARG, "cmi_linear_w8a8_bf16: null pointer");
    int8_t *xq;
    float *xs;
    if (const int rc = split_workspace("cmi_linear_w8a8_bf16", workspace, workspace_bytes, M, K, &xq, &xs)) return rc;
    // whatever the workspace holds beyond the quantised rows is room for split-K: 256 arrival
    // counters, cleared by the quantiser's launch, then partial tiles
    const size_t base = cmi_linear_workspace_bytes(M, K), counters = round_up(sizeof(int) * ARRIVALS);
    int *arrivals = nullptr;
    void *partials = nullptr;
    size_t partial_bytes = 0;
    if (workspace_bytes > base + counters && gemm_w8a8_split_bytes(M, N, K)) {
        arrivals = reinterpret_cast<int *>(static_cast<unsigned char *>(workspace) + base);
        partials = static_cast<unsigned char *>(workspace) + base + counters;
        partial_bytes = workspace_bytes - base - counters;
    }
    if (const int rc = quant_act_i8_and_clear(x, xq, xs, M, K, arrivals, arrivals ? ARRIVALS : 0, stream)) return rc;
    return gemm_w8a8_split(xq, wq, xs, ws, y, nullptr, M, N, K, ldy, arrivals, partials, partial_bytes, stream);
}

extern "C" int cmi_linear_w4a8_bf16(const uint8_t *w4, const float *ws, const void *x, void *y, int M, int N, int K,
                                    int gs, void *workspace, size_t workspace_bytes, void *stream) {
    CMI_REQUIRE(M >= 0 && N >= 1 && K >= 1, CMI_E_ARG, "cmi_linear_w4a8_bf16: bad shape M=%d N=%d K=%d", M, N, K);
    if (M == 0) return CMI_OK;
    CMI_REQUIRE(w4 && ws && x && y, CMI_E_ARG, "cmi_linear_w4a8_bf16: null pointer");
    const int Kd = cmi_w4_device_k(K, gs);
    CMI_REQUIRE(Kd > 0, CMI_E_UNSUPPORTED, "cmi_linear_w4a8_bf16: group size %d, the kernels are built for 64, 128 and 256", gs);
    int8_t *xq;
    float *xs;
    if (const int rc = split_workspace("cmi_linear_w4a8_bf16", workspace, workspace_bytes, M, Kd, &xq, &xs)) return rc;
    return linear_w4a8_rows(w4, ws, x, y, M, N, K, gs, xq, xs, stream);
}
