// Embedding lookup on quantized weights: gather rows by token id and dequantise only those
// rows to bf16.  The tied input embedding / lm_head matrix is read whole by the projection
// (the largest GEMV of a decode step) but a lookup touches a few rows of it, so the gather
// works on the stored int8 / int4 bytes and writes bf16 once.
//   int8: out[t,k] = bf16(float(wq[id,k]) * scale[id])                (one fp32 multiply)
//   int4: out[t,k] = bf16(float(code(id,k) - 8) * scale[id, k/128])   (device layout of cmi_w4_repack)
// One workgroup per looked-up row.  An id outside [0, N) cannot be reported from the device
// without a synchronisation; its output row is filled with bf16 NaN so that it cannot pass for
// an embedding.
#include "common.hpp"

namespace {

using namespace cmi;

constexpr int THREADS = 256;
constexpr uint32_t BF16_NAN2 = 0x7fc07fc0u;

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// K % 16 == 0: a thread turns 16 int8 into 16 bf16 (16-byte load, two 16-byte stores).
__global__ void __launch_bounds__(THREADS)
embed_rows_i8_kernel(const int8_t *__restrict__ wq, const float *__restrict__ ws, const int64_t *__restrict__ ids,
                     uint16_t *__restrict__ out, int N, int K) {
    const int t = blockIdx.x;
    const int64_t id = ids[t];
    uint4 *orow = reinterpret_cast<uint4 *>(out + (size_t)t * K);
    const int nvec = K / 16;
    if (id < 0 || id >= N) {
        for (int i = threadIdx.x; i < nvec * 2; i += THREADS) orow[i] = make_uint4(BF16_NAN2, BF16_NAN2, BF16_NAN2, BF16_NAN2);
        return;
    }
    const float sc = ws[id];
    const uint4 *wrow = reinterpret_cast<const uint4 *>(wq + (size_t)id * K);
    for (int i = threadIdx.x; i < nvec; i += THREADS) {
        const uint4 v = wrow[i];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float b0 = (float)(int8_t)(w[j] & 0xff), b1 = (float)(int8_t)((w[j] >> 8) & 0xff);
            const float b2 = (float)(int8_t)((w[j] >> 16) & 0xff), b3 = (float)(int8_t)(w[j] >> 24);
            o[2 * j] = pack2(__fmul_rn(b0, sc), __fmul_rn(b1, sc));
            o[2 * j + 1] = pack2(__fmul_rn(b2, sc), __fmul_rn(b3, sc));
        }
        orow[2 * i] = make_uint4(o[0], o[1], o[2], o[3]);
        orow[2 * i + 1] = make_uint4(o[4], o[5], o[6], o[7]);
    }
}

// Any K (tail and unaligned rows).
__global__ void __launch_bounds__(THREADS)
embed_rows_i8_scalar(const int8_t *__restrict__ wq, const float *__restrict__ ws, const int64_t *__restrict__ ids,
                     uint16_t *__restrict__ out, int N, int K) {
    const int t = blockIdx.x;
    const int64_t id = ids[t];
    uint16_t *orow = out + (size_t)t * K;
    const bool ok = id >= 0 && id < N;
    const float sc = ok ? ws[id] : 0.f;
    for (int k = threadIdx.x; k < K; k += THREADS)
        orow[k] = ok ? (uint16_t)f32_to_bf16_bits(__fmul_rn((float)wq[(size_t)id * K + k], sc)) : (uint16_t)0x7fc0;
}

// Device int4 layout: row n is K/2 bytes; in 32-bit word i byte b holds code(8i+b) in its low
// nibble and code(8i+4+b) in its high nibble.  A thread expands one 16-byte load = 32 codes of
// one 128-element group into 32 bf16 (four 16-byte stores).  K % 128 == 0.
__global__ void __launch_bounds__(THREADS)
embed_rows_w4_kernel(const uint8_t *__restrict__ w4, const float *__restrict__ ws, const int64_t *__restrict__ ids,
                     uint16_t *__restrict__ out, int N, int K) {
    const int t = blockIdx.x;
    const int64_t id = ids[t];
    uint4 *orow = reinterpret_cast<uint4 *>(out + (size_t)t * K);
    const int nvec = K / 32, G = K / 128;
    if (id < 0 || id >= N) {
        for (int i = threadIdx.x; i < nvec * 4; i += THREADS) orow[i] = make_uint4(BF16_NAN2, BF16_NAN2, BF16_NAN2, BF16_NAN2);
        return;
    }
    const uint4 *wrow = reinterpret_cast<const uint4 *>(w4 + (size_t)id * (K / 2));
    const float *srow = ws + (size_t)id * G;
    for (int i = threadIdx.x; i < nvec; i += THREADS) {
        const uint4 v = wrow[i];
        const float sc = srow[i >> 2];  // 4 vectors of 32 codes per group of 128
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {  // word j: codes 8j .. 8j+7 of this vector
            float c[8];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                c[b] = (float)((int)((w[j] >> (8 * b)) & 15) - 8);
                c[4 + b] = (float)((int)((w[j] >> (8 * b + 4)) & 15) - 8);
            }
            orow[4 * i + j] = make_uint4(pack2(__fmul_rn(c[0], sc), __fmul_rn(c[1], sc)),
                                         pack2(__fmul_rn(c[2], sc), __fmul_rn(c[3], sc)),
                                         pack2(__fmul_rn(c[4], sc), __fmul_rn(c[5], sc)),
                                         pack2(__fmul_rn(c[6], sc), __fmul_rn(c[7], sc)));
        }
    }
}

// Any group size the device layout takes and any K: a thread expands one 32-bit word (8 codes);
// rows are Kd / 2 bytes apart (Kd: K padded to whole groups and steps), the output has K columns.
__global__ void __launch_bounds__(THREADS)
embed_rows_w4_general(const uint8_t *__restrict__ w4, const float *__restrict__ ws, const int64_t *__restrict__ ids,
                      uint16_t *__restrict__ out, int N, int K, int Kd, int gs) {
    const int t = blockIdx.x;
    const int64_t id = ids[t];
    uint16_t *orow = out + (size_t)t * K;
    if (id < 0 || id >= N) {
        for (int k = threadIdx.x; k < K; k += THREADS) orow[k] = 0x7fc0;
        return;
    }
    const uint32_t *wrow = reinterpret_cast<const uint32_t *>(w4 + (size_t)id * (Kd / 2));
    const float *srow = ws + (size_t)id * (Kd / gs);
    for (int i = threadIdx.x; i * 8 < K; i += THREADS) {
        const uint32_t w = wrow[i];
        const float sc = srow[(8 * i) / gs];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int lo = 8 * i + b, hi = lo + 4;
            if (lo < K) orow[lo] = (uint16_t)f32_to_bf16_bits(__fmul_rn((float)((int)((w >> (8 * b)) & 15) - 8), sc));
            if (hi < K) orow[hi] = (uint16_t)f32_to_bf16_bits(__fmul_rn((float)((int)((w >> (8 * b + 4)) & 15) - 8), sc));
        }
    }
}

}  // namespace

extern "C" int cmi_embed_rows_i8(const int8_t *wq, const float *ws, const int64_t *ids, void *out, int T, int N,
                                 int K, void *stream) {
    CMI_REQUIRE(T >= 0 && N >= 1 && K >= 1, CMI_E_ARG, "cmi_embed_rows_i8: bad shape T=%d N=%d K=%d", T, N, K);
    if (T == 0) return CMI_OK;
    CMI_REQUIRE(wq && ws && ids && out, CMI_E_ARG, "cmi_embed_rows_i8: null pointer");
    CMI_REQUIRE(aligned(ids, 8) && aligned(out, 2), CMI_E_ARG, "cmi_embed_rows_i8: ids must be 8-byte aligned int64");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (K % 16 == 0 && aligned(wq, 16) && aligned(out, 16))
        embed_rows_i8_kernel<<<dim3(T), dim3(THREADS), 0, st>>>(wq, ws, ids, static_cast<uint16_t *>(out), N, K);
    else
        embed_rows_i8_scalar<<<dim3(T), dim3(THREADS), 0, st>>>(wq, ws, ids, static_cast<uint16_t *>(out), N, K);
    return check_launch("cmi_embed_rows_i8");
}

extern "C" int cmi_embed_rows_w4(const uint8_t *w4, const float *ws, const int64_t *ids, void *out, int T, int N,
                                 int K, int gs, void *stream) {
    CMI_REQUIRE(T >= 0 && N >= 1 && K >= 1, CMI_E_ARG, "cmi_embed_rows_w4: bad shape T=%d N=%d K=%d", T, N, K);
    if (T == 0) return CMI_OK;
    CMI_REQUIRE(w4 && ws && ids && out, CMI_E_ARG, "cmi_embed_rows_w4: null pointer");
    const int Kd = cmi_w4_device_k(K, gs);
    CMI_REQUIRE(Kd > 0, CMI_E_UNSUPPORTED, "cmi_embed_rows_w4: group size %d, the device layout is built for 64, 128 and 256", gs);
    CMI_REQUIRE(aligned(w4, 16) && aligned(out, 2) && aligned(ids, 8), CMI_E_ARG,
                "cmi_embed_rows_w4: w4 must be 16-byte aligned, ids 8-byte aligned int64");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (gs == 128 && Kd == K && aligned(out, 16))
        embed_rows_w4_kernel<<<dim3(T), dim3(THREADS), 0, st>>>(w4, ws, ids, static_cast<uint16_t *>(out), N, K);
    else
        embed_rows_w4_general<<<dim3(T), dim3(THREADS), 0, st>>>(w4, ws, ids, static_cast<uint16_t *>(out), N, K, Kd, gs);
    return check_launch("cmi_embed_rows_w4");
}
