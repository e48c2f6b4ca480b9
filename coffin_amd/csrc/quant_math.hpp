// Arithmetic of the per-token int8 activation quantiser, shared by the stand-alone
// kernel and by kernels that quantise their activations on the fly.  The scale
// and the rounding follow the torch statement bit for bit: scale =
// max(absmax, 1e-5) / 127, IEEE fp32 division by the scale (not a reciprocal
// multiply), round-half-even, clamp to +-127.
#pragma once

#include "common.hpp"

namespace cmi {

__device__ __forceinline__ float quant_scale(float absmax) { return fmaxf(absmax, 1e-5f) / 127.0f; }

__device__ __forceinline__ float absmax8(const uint4 &v, float amax) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        amax = fmaxf(amax, fabsf(bf16_bits_to_f32(w[i] & 0xffffu)));
        amax = fmaxf(amax, fabsf(__uint_as_float(w[i] & 0xffff0000u)));
    }
    return amax;
}

__device__ __forceinline__ uint32_t quant1(float x, float sc) {
    float q = rintf(__fdiv_rn(x, sc));
    q = fminf(fmaxf(q, -127.f), 127.f);
    return (uint32_t)((int)q) & 0xffu;
}

__device__ __forceinline__ uint2 quant8(const uint4 &v, float sc) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t b[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        b[2 * i] = quant1(bf16_bits_to_f32(w[i] & 0xffffu), sc);
        b[2 * i + 1] = quant1(__uint_as_float(w[i] & 0xffff0000u), sc);
    }
    uint2 o;
    o.x = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
    o.y = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
    return o;
}

}  // namespace cmi
