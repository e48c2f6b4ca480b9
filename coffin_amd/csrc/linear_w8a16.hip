// int8 weight-only projection of any number of bf16 rows in one call, with the kernel family as
// an argument: the dot-product GEMV (a row's bits are those of the single-row call) or the
// matrix-pipe GEMV (a row's bits depend on K only, not on the dot-product kernel's).  The batch is
// cut into the launches the family takes; every piece goes to the same family, so a row's bits
// never depend on where the batch was cut.
#include "common.hpp"

extern "C" int cmi_linear_w8a16(const int8_t *wq, const float *ws, const void *x, void *y, int M, int N, int K,
                                int family, void *stream) {
    using namespace cmi;
    CMI_REQUIRE(M >= 0 && N >= 1 && K >= 1, CMI_E_ARG, "cmi_linear_w8a16: bad shape M=%d N=%d K=%d", M, N, K);
    CMI_REQUIRE(family == CMI_FAMILY_DOT || family == CMI_FAMILY_MFMA, CMI_E_ARG,
                "cmi_linear_w8a16: family=%d, expected CMI_FAMILY_DOT (0) or CMI_FAMILY_MFMA (1)", family);
    if (M == 0) return CMI_OK;
    CMI_REQUIRE(wq && ws && x && y, CMI_E_ARG, "cmi_linear_w8a16: null pointer");
    const int step = family == CMI_FAMILY_MFMA ? 64 : 16;
    const uint16_t *xr = static_cast<const uint16_t *>(x);
    uint16_t *yr = static_cast<uint16_t *>(y);
    for (int lo = 0; lo < M; lo += step) {
        const int m = M - lo < step ? M - lo : step;
        const int rc = family == CMI_FAMILY_MFMA
                           ? cmi_gemv_w8a16_mfma(wq, ws, xr + (size_t)lo * K, yr + (size_t)lo * N, m, N, K, stream)
                           : cmi_gemv_w8a16(wq, ws, xr + (size_t)lo * K, yr + (size_t)lo * N, m, N, K, stream);
        if (rc) return rc;
    }
    return CMI_OK;
}

extern "C" long long cmi_stream_capture_id(void *stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    if (hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &status, &id) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    if (status != hipStreamCaptureStatusActive) return 0;
    return (long long)(id & 0x7fffffffffffffffull) + 1;  // never 0 while a capture is active
}
