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

// 1.5 * 2^23: q + MAGIC has a unit in the last place of 1 for |q| < 2^22, so the sum is q rounded to
// the nearest integer (ties to even) and its low mantissa bits are that integer in two's complement.
constexpr float ROUND_MAGIC = 12582912.0f;

// The quantised value of one element in the LOW BYTE of the result (the other bytes are not
// zero: callers pick the byte out with a permute or a mask).  Finite rows: corrected quotient,
// rounding and narrowing in one addition, no clamp -- |x / scale| <= 127 up to one rounding, so
// the rounded value cannot leave [-127, 127] (part of the exhaustive CPU check).  Rows without a
// finite scale divide, round and clamp as the reference statement does.
__device__ __forceinline__ uint32_t quant1_lowbyte(float x, const RowScale &s) {
    if (s.rc != 0.f) {
        const float q0 = __fmul_rn(x, s.rc);
        const float e = __fmaf_rn(-q0, s.sc, x);
        const float t = __fmaf_rn(e, s.rc, q0);
        return __float_as_uint(__fadd_rn(t, ROUND_MAGIC));
    }
    float q = rintf(__fdiv_rn(x, s.sc));
    q = fminf(fmaxf(q, -127.f), 127.f);
    return (uint32_t)((int)q);
}

__device__ __forceinline__ uint32_t quant1(float x, const RowScale &s) { return quant1_lowbyte(x, s) & 0xffu; }

__device__ __forceinline__ uint2 quant8(const uint4 &v, const RowScale &s) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t b[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        b[2 * i] = quant1_lowbyte(bf16_bits_to_f32(w[i] & 0xffffu), s);
        b[2 * i + 1] = quant1_lowbyte(__uint_as_float(w[i] & 0xffff0000u), s);
    }
    // low bytes of four results -> one dword: two permutes gather pairs, a third joins them
    uint2 o;
    o.x = __builtin_amdgcn_perm(__builtin_amdgcn_perm(b[3], b[2], 0x0c0c0400u), __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u),
                                0x05040100u);
    o.y = __builtin_amdgcn_perm(__builtin_amdgcn_perm(b[7], b[6], 0x0c0c0400u), __builtin_amdgcn_perm(b[5], b[4], 0x0c0c0400u),
                                0x05040100u);
    return o;
}

}  // namespace cmi
