// Per-token symmetric int8 activation quantiser (bf16 in, int8 + fp32 scale out).
//
// One workgroup per row.  The row is read once from HBM with 16-byte loads and
// kept in registers across the absmax reduction when it fits (VPT vectors per
// thread), so HBM traffic is the algorithmic 2 B in + 1 B out per element.
// The scale and the rounding follow the torch spec bit for bit: IEEE fp32
// division by the scale (not a reciprocal multiply), round-half-even, clamp.
#include "quant_math.hpp"

namespace {

using namespace cmi;

constexpr int QUANT_THREADS = 256;

// Block-wide max of non-negative values; every thread returns the result.
__device__ __forceinline__ float block_max(float v, float *smem) {
    v = wave_max_to_lane63(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 63) smem[wave] = v;
    __syncthreads();
    float r = smem[0];
#pragma unroll
    for (int i = 1; i < QUANT_THREADS / 64; ++i) r = fmaxf(r, smem[i]);
    return r;
}

// K % 8 == 0, rows 16-byte aligned.  VPT > 0: the row fits in VPT vectors per
// thread and stays in registers; VPT == 0: generic, second pass re-reads.
// zero / n_zero: a few ints of the caller's that the first workgroup clears on the way (the
// arrival counters of a split-K GEMM that follows in the stream), or null / 0.
template <int VPT>
__global__ void __launch_bounds__(QUANT_THREADS)
quant_act_i8_vec(const uint4 *__restrict__ x, uint2 *__restrict__ q, float *__restrict__ s,
                 int nvec, int *__restrict__ zero, int n_zero) {
    __shared__ float smem[QUANT_THREADS / 64];
    const int row = blockIdx.x;
    if (row == 0)
        for (int i = threadIdx.x; i < n_zero; i += QUANT_THREADS) zero[i] = 0;
    const uint4 *xr = x + (size_t)row * nvec;
    uint2 *qr = q + (size_t)row * nvec;
    float amax = 0.f;
    if constexpr (VPT > 0) {
        uint4 v[VPT];
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int idx = threadIdx.x + i * QUANT_THREADS;
            v[i] = idx < nvec ? xr[idx] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) amax = absmax8(v[i], amax);
        amax = block_max(amax, smem);
        const RowScale rs = row_scale(amax);
        const float sc = rs.sc;
        if (threadIdx.x == 0) s[row] = sc;
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int idx = threadIdx.x + i * QUANT_THREADS;
            if (idx < nvec) qr[idx] = quant8(v[i], rs);
        }
    } else {
        for (int idx = threadIdx.x; idx < nvec; idx += QUANT_THREADS) amax = absmax8(xr[idx], amax);
        amax = block_max(amax, smem);
        const RowScale rs = row_scale(amax);
        const float sc = rs.sc;
        if (threadIdx.x == 0) s[row] = sc;
        for (int idx = threadIdx.x; idx < nvec; idx += QUANT_THREADS) qr[idx] = quant8(xr[idx], rs);
    }
}

// Any K, any alignment; q rows have pitch ldq >= K and the tail K .. ldq-1 is cleared.
__global__ void __launch_bounds__(QUANT_THREADS)
quant_act_i8_scalar(const uint16_t *__restrict__ x, int8_t *__restrict__ q,
                    float *__restrict__ s, int K, int ldq, int *__restrict__ zero, int n_zero) {
    __shared__ float smem[QUANT_THREADS / 64];
    const int row = blockIdx.x;
    if (row == 0)
        for (int i = threadIdx.x; i < n_zero; i += QUANT_THREADS) zero[i] = 0;
    const uint16_t *xr = x + (size_t)row * K;
    int8_t *qr = q + (size_t)row * ldq;
    for (int k = K + threadIdx.x; k < ldq; k += QUANT_THREADS) qr[k] = 0;
    float amax = 0.f;
    for (int k = threadIdx.x; k < K; k += QUANT_THREADS)
        amax = fmaxf(amax, fabsf(bf16_bits_to_f32(xr[k])));
    amax = block_max(amax, smem);
    const RowScale rs = row_scale(amax);
    const float sc = rs.sc;
    if (threadIdx.x == 0) s[row] = sc;
    for (int k = threadIdx.x; k < K; k += QUANT_THREADS)
        qr[k] = (int8_t)quant1(bf16_bits_to_f32(xr[k]), rs);
}

}  // namespace

int cmi::quant_act_i8_and_clear(const void *x, int8_t *q, float *s, int M, int K, int *zero, int n_zero,
                                void *stream) {
    CMI_REQUIRE(M >= 0 && K > 0, CMI_E_ARG, "cmi_quant_act_i8: bad shape M=%d K=%d", M, K);
    if (M == 0) return CMI_OK;  // an empty batch has no storage to point at
    CMI_REQUIRE(x && q && s, CMI_E_ARG, "cmi_quant_act_i8: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(M), block(QUANT_THREADS);
    if (K % 8 == 0 && aligned(x, 16) && aligned(q, 8)) {
        const int nvec = K / 8;
        const uint4 *xv = static_cast<const uint4 *>(x);
        uint2 *qv = reinterpret_cast<uint2 *>(q);
        const int vpt = (nvec + QUANT_THREADS - 1) / QUANT_THREADS;
        if (vpt <= 1) quant_act_i8_vec<1><<<grid, block, 0, st>>>(xv, qv, s, nvec, zero, n_zero);
        else if (vpt <= 2) quant_act_i8_vec<2><<<grid, block, 0, st>>>(xv, qv, s, nvec, zero, n_zero);
        else if (vpt <= 4) quant_act_i8_vec<4><<<grid, block, 0, st>>>(xv, qv, s, nvec, zero, n_zero);
        else if (vpt <= 8) quant_act_i8_vec<8><<<grid, block, 0, st>>>(xv, qv, s, nvec, zero, n_zero);
        else if (vpt <= 16) quant_act_i8_vec<16><<<grid, block, 0, st>>>(xv, qv, s, nvec, zero, n_zero);
        else quant_act_i8_vec<0><<<grid, block, 0, st>>>(xv, qv, s, nvec, zero, n_zero);
    } else {
        quant_act_i8_scalar<<<grid, block, 0, st>>>(static_cast<const uint16_t *>(x), q, s, K, K, zero, n_zero);
    }
    return check_launch("cmi_quant_act_i8");
}

int cmi::quant_act_i8_padded(const void *x, int8_t *q, float *s, int M, int K, int ldq, void *stream) {
    if (ldq == K) return quant_act_i8_and_clear(x, q, s, M, K, nullptr, 0, stream);
    CMI_REQUIRE(M >= 0 && K > 0 && ldq > K, CMI_E_ARG, "cmi_quant_act_i8: bad shape M=%d K=%d pitch=%d", M, K, ldq);
    if (M == 0) return CMI_OK;
    CMI_REQUIRE(x && q && s, CMI_E_ARG, "cmi_quant_act_i8: null pointer");
    quant_act_i8_scalar<<<dim3(M), dim3(QUANT_THREADS), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint16_t *>(x), q, s, K, ldq, nullptr, 0);
    return check_launch("cmi_quant_act_i8");
}

extern "C" int cmi_quant_act_i8(const void *x, int8_t *q, float *s, int M, int K, void *stream) {
    return cmi::quant_act_i8_and_clear(x, q, s, M, K, nullptr, 0, stream);
}
