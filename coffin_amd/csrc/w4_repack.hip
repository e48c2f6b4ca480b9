// One-time re-layout of a group-quantised int4 weight for the gfx950 kernels.
//
// Contract storage is K-major: packed[k/2, n] holds code(k even) in the low and
// code(k+1) in the high nibble, scale[g, n] one fp32 per group and output
// channel.  The GEMV/GEMM kernels stream each output row along K with 16-byte
// loads and feed v_dot4_i32_i8 / int8 MFMA four k at a time, so the device copy
// is N-major and re-interleaved: in every 32-bit word (8 consecutive k starting
// at k0) byte b holds code(k0+b) in its low and code(k0+4+b) in its high
// nibble.  `w & 0x0F0F0F0F` and `(w >> 4) & 0x0F0F0F0F` then are the four-byte
// operands for k0..k0+3 and k0+4..k0+7.
#include "common.hpp"

#include <climits>

namespace {

using namespace cmi;

// One thread per output word; n fastest so the K-major reads coalesce.  Source rows beyond
// src_rows (device rows are padded to whole groups and whole 128-element steps) read as code 8.
__global__ void __launch_bounds__(256)
w4_repack_kernel(const uint8_t *__restrict__ packed, uint32_t *__restrict__ w4, int N, int words, int src_rows) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int wi = blockIdx.y;
    if (n >= N) return;
    const uint8_t *src = packed + (size_t)(wi * 4) * N + n;
    uint32_t b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) b[i] = wi * 4 + i < src_rows ? (uint32_t)src[(size_t)i * N] : 0x88u;
    // b0 = c0|c1<<4, b1 = c2|c3<<4, b2 = c4|c5<<4, b3 = c6|c7<<4
    const uint32_t o0 = (b[0] & 15u) | ((b[2] & 15u) << 4);
    const uint32_t o1 = (b[0] >> 4) | ((b[2] >> 4) << 4);
    const uint32_t o2 = (b[1] & 15u) | ((b[3] & 15u) << 4);
    const uint32_t o3 = (b[1] >> 4) | ((b[3] >> 4) << 4);
    w4[(size_t)n * words + wi] = o0 | (o1 << 8) | (o2 << 16) | (o3 << 24);
}

// Groups beyond the source's (padding up to a whole 128-element step) get the scale 0.
__global__ void __launch_bounds__(256)
scale_transpose_kernel(const float *__restrict__ scale, float *__restrict__ ws, int N, int G, int src_groups) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int g = blockIdx.y;
    if (n < N) ws[(size_t)n * G + g] = g < src_groups ? scale[(size_t)g * N + n] : 0.f;
}

}  // namespace

extern "C" int cmi_w4_device_k(int K, int gs) {
    if (K < 1 || (gs != 64 && gs != 128 && gs != 256)) return 0;
    const int unit = gs > 128 ? gs : 128;
    if (K > INT32_MAX - unit) return 0;
    return (K + unit - 1) / unit * unit;
}

extern "C" int cmi_w4_repack(const uint8_t *packed, const float *scale, uint8_t *w4, float *ws,
                             int N, int K, int gs, void *stream) {
    CMI_REQUIRE(packed && scale && w4 && ws, CMI_E_ARG, "cmi_w4_repack: null pointer");
    CMI_REQUIRE(N >= 1 && K >= 1 && gs >= 1, CMI_E_ARG, "cmi_w4_repack: bad shape N=%d K=%d gs=%d", N, K, gs);
    const int Kd = cmi_w4_device_k(K, gs);
    CMI_REQUIRE(Kd > 0, CMI_E_UNSUPPORTED, "cmi_w4_repack: group size %d, the kernels are built for 64, 128 and 256", gs);
    CMI_REQUIRE(aligned(w4, 16), CMI_E_ARG, "cmi_w4_repack: w4 must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the source holds whole groups (and an even number of codes): w4a8_weights.py:28-50
    const int src_groups = (K + gs - 1) / gs, src_rows = (src_groups * gs + 1) / 2;
    const int words = Kd / 8, G = Kd / gs;
    CMI_REQUIRE(words <= 65535 && G <= 65535, CMI_E_UNSUPPORTED, "cmi_w4_repack: K=%d too large", K);
    const dim3 block(256);
    w4_repack_kernel<<<dim3((N + 255) / 256, words), block, 0, st>>>(
        packed, reinterpret_cast<uint32_t *>(w4), N, words, src_rows);
    scale_transpose_kernel<<<dim3((N + 255) / 256, G), block, 0, st>>>(scale, ws, N, G, src_groups);
    return check_launch("cmi_w4_repack");
}
