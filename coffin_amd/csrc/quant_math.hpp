// Arithmetic of the per-token int8 activation quantiser, shared by the stand-alone
// kernel and by kernels that quantise their activations on the fly.  The result
// follows the torch statement bit for bit: scale = max(absmax, 1e-5) / 127,
// q = clamp(rint(x / scale), +-127) with an IEEE fp32 division.
//
// The division is not executed per element.  With rc = 1 / scale (one IEEE
// division per row) the kernels form
//     q0 = x * rc;   e = fma(-q0, scale, x);   q1 = fma(e, rc, q0)
// and round q1.  A bare x * rc rounds differently from x / scale on some inputs;
// the corrected q1 gives the same integer for every finite bf16 x and every
// scale a row of bf16 values can have -- checked pair by pair (about 10^9 of
// them) on the CPU, not argued.  Rows whose scale is not finite keep the division.
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

// A row's scale and its reciprocal; rc == 0 marks a row that takes the division path.
struct RowScale {
    float sc, rc;
};

__device__ __forceinline__ RowScale row_scale(float absmax) {
    RowScale s;
    s.sc = quant_scale(absmax);
    s.rc = s.sc < __builtin_inff() ? __fdiv_rn(1.0f, s.sc) : 0.f;  // false for NaN too
    return s;
}

__device__ __forceinline__ uint32_t quant1(float x, const RowScale &s) {
    float t;
    if (s.rc != 0.f) {
        const float q0 = __fmul_rn(x, s.rc);
        const float e = __fmaf_rn(-q0, s.sc, x);
        t = __fmaf_rn(e, s.rc, q0);
    } else {
        t = __fdiv_rn(x, s.sc);
    }
    float q = rintf(t);
    q = fminf(fmaxf(q, -127.f), 127.f);
    return (uint32_t)((int)q) & 0xffu;
}

__device__ __forceinline__ uint2 quant8(const uint4 &v, const RowScale &s) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t b[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        b[2 * i] = quant1(bf16_bits_to_f32(w[i] & 0xffffu), s);
        b[2 * i + 1] = quant1(__uint_as_float(w[i] & 0xffff0000u), s);
    }
    uint2 o;
    o.x = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
    o.y = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
    return o;
}

}  // namespace cmi
