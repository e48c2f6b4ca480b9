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

namespace {

using namespace cmi;

// One thread per output word; n fastest so the K-major reads coalesce.
__global__ void __launch_bounds__(256)
w4_repack_kernel(const uint8_t *__restrict__ packed, uint32_t *__restrict__ w4, int N, int words) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int wi = blockIdx.y;
    if (n >= N) return;
    const uint8_t *src = packed + (size_t)(wi * 4) * N + n;
    const uint32_t b0 = src[0], b1 = src[(size_t)N], b2 = src[(size_t)2 * N], b3 = src[(size_t)3 * N];
    // b0 = c0|c1<<4, b1 = c2|c3<<4, b2 = c4|c5<<4, b3 = c6|c7<<4
    const uint32_t o0 = (b0 & 15u) | ((b2 & 15u) << 4);
    const uint32_t o1 = (b0 >> 4) | ((b2 >> 4) << 4);
    const uint32_t o2 = (b1 & 15u) | ((b3 & 15u) << 4);
    const uint32_t o3 = (b1 >> 4) | ((b3 >> 4) << 4);
    w4[(size_t)n * words + wi] = o0 | (o1 << 8) | (o2 << 16) | (o3 << 24);
}

__global__ void __launch_bounds__(256)
scale_transpose_kernel(const float *__restrict__ scale, float *__restrict__ ws, int N, int G) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int g = blockIdx.y;
    if (n < N) ws[(size_t)n * G + g] = scale[(size_t)g * N + n];
}

}  // namespace

extern "C" int cmi_w4_repack(const uint8_t *packed, const float *scale, uint8_t *w4, float *ws,
                             int N, int K, int gs, void *stream) {
    CMI_REQUIRE(packed && scale && w4 && ws, CMI_E_ARG, "cmi_w4_repack: null pointer");
    CMI_REQUIRE(N >= 1 && K >= 32 && gs >= 32, CMI_E_ARG, "cmi_w4_repack: bad shape N=%d K=%d gs=%d", N, K, gs);
    CMI_REQUIRE(K % 32 == 0 && gs % 32 == 0 && K % gs == 0, CMI_E_UNSUPPORTED,
                "cmi_w4_repack: K=%d and group size %d must be multiples of 32 and K a multiple of the group size", K, gs);
    CMI_REQUIRE(aligned(w4, 16), CMI_E_ARG, "cmi_w4_repack: w4 must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int words = K / 8, G = K / gs;
    CMI_REQUIRE(words <= 65535 && G <= 65535, CMI_E_UNSUPPORTED, "cmi_w4_repack: K=%d too large", K);
    const dim3 block(256);
    w4_repack_kernel<<<dim3((N + 255) / 256, words), block, 0, st>>>(
        packed, reinterpret_cast<uint32_t *>(w4), N, words);
    scale_transpose_kernel<<<dim3((N + 255) / 256, G), block, 0, st>>>(scale, ws, N, G);
    return check_launch("cmi_w4_repack");
}
