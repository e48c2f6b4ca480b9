// Arithmetic shared by the int8 weight-only GEMV kernels: the canonical summation order's
// blocking of K and the exact int8 -> packed-bf16 widening.  Every kernel that includes this
// produces the same bits for the same (weight row, activation row).
#pragma once

#include "common.hpp"

namespace cmi {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Segments per unit: the largest of 4,3,2,1 that pads K by at most a fifth.
__host__ __device__ inline int unit_segments(int nseg) {
    for (int u = 4; u > 1; --u) {
        const int padded = (nseg + u - 1) / u * u;
        if ((padded - nseg) * 5 <= padded) return u;
    }
    return 1;
}

// Four int8 in one dword -> two packed-bf16 pairs (k, k+1) and (k+2, k+3).
__device__ __forceinline__ void widen4(uint32_t w, bf16x2_t &lo, bf16x2_t &hi) {
    const float f0 = (float)(int8_t)(w);
    const float f1 = (float)(int8_t)(w >> 8);
    const float f2 = (float)(int8_t)(w >> 16);
    const float f3 = (float)(int8_t)(w >> 24);
    // Integers up to 127 occupy only the upper 16 bits of their fp32 pattern,
    // so taking the high halves is an exact conversion to bf16.
    const uint32_t p0 = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
    const uint32_t p1 = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
    lo = __builtin_bit_cast(bf16x2_t, p0);
    hi = __builtin_bit_cast(bf16x2_t, p1);
}


// One 16-element chunk of a lane's chain: eight chained two-element dot products, k ascending.
__device__ __forceinline__ float chain_chunk(float v, const u32x4 &w, const uint4 &x0, const uint4 &x1) {
    bf16x2_t wb[8];
    widen4(w.x, wb[0], wb[1]);
    widen4(w.y, wb[2], wb[3]);
    widen4(w.z, wb[4], wb[5]);
    widen4(w.w, wb[6], wb[7]);
    const uint32_t xv[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
    for (int i = 0; i < 8; ++i)
        v = __builtin_amdgcn_fdot2_f32_bf16(wb[i], __builtin_bit_cast(bf16x2_t, xv[i]), v, false);
    return v;
}

}  // namespace cmi
