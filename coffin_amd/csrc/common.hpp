// Shared device helpers and host-side status plumbing for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

#include "../../include/coffin_mi355.h"

namespace cmi {

// ---------------------------------------------------------------- host status
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);
// Raise a kernel's dynamic-LDS limit to `bytes` on the current device, once per device
// (`devices`: one bit per device ordinal, owned by the call site).  CMI_OK or CMI_E_HIP.
int reserve_lds(const void *kernel, int bytes, std::atomic<uint64_t> &devices, const char *who);
// CUs of the current device (0: it cannot be read); cached per device.
int compute_units();

// Kernel-selection overrides (cmi_set_option / CMI_GEMM_TILE, CMI_GEMV_WHOLEROW read once).
int option_gemm_tile();      // 0 = the library chooses, else 64 / 128 / 192 / 256 / 320 / 6464 / 128192
int option_gemv_wholerow();  // -1 = the library chooses, 0 = never, 1 = where it can
int option_w4_decode_waves();  // 0 = the library chooses, else 4 or 16 wavefronts per workgroup
int option_w4_decode_chain();  // 0 = the library chooses, 1 = never, else a variant code of gemv_w4a8_chain

#define CMI_REQUIRE(cond, code, ...)                 \
    do {                                             \
        if (!(cond)) return cmi::fail(code, __VA_ARGS__); \
    } while (0)

// gemm_mfma.hip: register-staged W8A8 GEMM for K % 64 != 0 (see gemm_w8a8.hip for the fast path).
int gemm_w8a8_generic(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws, void *y,
                      int32_t *acc_out, int M, int N, int K, int ldy, void *stream);
// gemm_w8a8_rows16.hip: W8A8 for up to 16 rows with the weight read once (K % 128 == 0,
// K <= 10240); CMI_E_UNSUPPORTED (no error text) outside that range.
int gemm_w8a8_rows16(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws, void *y,
                     int32_t *acc_out, int M, int N, int K, int ldy, void *stream);
// gemm_w8a8.hip: cmi_gemm_w8a8 with room for split-K (arrival counters, 256 ints, zero; partial
// tiles, gemm_w8a8_split_bytes(M, N, K) bytes or fewer: the kernel choice adapts); both null = no split.
int gemm_w8a8_split(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws, void *y,
                    int32_t *acc_out, int M, int N, int K, int ldy, int *arrivals, void *partials,
                    size_t partial_bytes, void *stream);
size_t gemm_w8a8_split_bytes(int M, int N, int K);
// quant_act_i8.hip: cmi_quant_act_i8 that also clears n_zero ints at `zero` (null / 0: none).
int quant_act_i8_and_clear(const void *x, int8_t *q, float *s, int M, int K, int *zero, int n_zero, void *stream);
// quant_act_i8.hip: the quantiser writing rows of pitch ldq >= K, the tail K .. ldq-1 cleared (rows
// of an int4 weight whose K is padded to whole groups on the device).
int quant_act_i8_padded(const void *x, int8_t *q, float *s, int M, int K, int ldq, void *stream);
// 16-row weight tiles per workgroup (1 or 2) that gemm_w8a8_rows16 uses for 17..128 rows.
int gemm_w8a8_rows_tiles(int N);

// gemv_w4a8_decode.hip: W4A8 GEMV for 1..4 rows, K <= 10240, from bf16 activations (x) or
// quantised ones (xq, xs); returns CMI_E_UNSUPPORTED (no error text) for other shapes.
int gemv_w4a8_decode(const uint8_t *w4, const float *ws, const void *x, const int8_t *xq, const float *xs,
                     void *y, int32_t *group_acc, int8_t *xq_out, float *xs_out, int M, int N, int K,
                     void *stream);
// gemv_w4a8_chain.hip: the same for 1..2 rows with the fp32 chain in registers; `variant` = lanes per
// weight row (8, 16) + 100 * wavefronts sharing a row (1, 2, 4, 8) + 10000 * wavefronts per workgroup
// (4, 8, 16); CMI_E_UNSUPPORTED (no error text) outside the variant's range.
int gemv_w4a8_chain(const uint8_t *w4, const float *ws, const void *x, const int8_t *xq, const float *xs,
                    void *y, int32_t *group_acc, int8_t *xq_out, float *xs_out, int M, int N, int K,
                    int variant, void *stream);
// gemv_w4a8_rows16.hip: W4A8 GEMV for up to 16 quantised rows (xq, xs) or up to 4 bf16 rows (x,
// quantised in the kernel), K <= 10240, integer sums on the matrix pipe; CMI_E_UNSUPPORTED (no error text) outside that range.
int gemv_w4a8_rows16(const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs, const void *x,
                     void *y, int32_t *group_acc, int8_t *xq_out, float *xs_out, int M, int N, int K,
                     void *stream);
// gemm_w4a8_ring.hip: W4A8 tile GEMM with a ring of LDS stages for launches of few tiles; tile =
// 6464 (64 x 64) or 64 (128 m x 64 n); arguments already checked.
int gemm_w4a8_ring(const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs, void *y, int M, int N,
                   int K, int tile, void *stream, int ldy = 0);  // ldy: row pitch of y (0: N)
// linear_bf16.hip: quantiser + W4A8 GEMV / GEMM (or the GEMV that quantises by itself where that
// is faster) on bf16 rows, with xq int8 [M,K] / xs fp32 [M] as staging; arguments already checked.
int linear_w4a8_rows(const uint8_t *w4, const float *ws, const void *x, void *y, int M, int N, int K, int gs,
                     int8_t *xq, float *xs, void *stream);
static inline bool aligned(const void *p, uintptr_t a) {
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

// ------------------------------------------------------------- device helpers
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef int v16i32 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t v) {
    return __uint_as_float(v << 16);
}

// fp32 -> bf16 bit pattern, round to nearest even (finite inputs).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

typedef float f32x2_t __attribute__((ext_vector_type(2)));

// Two fp32 -> packed bf16 (lo in the low half), round to nearest even, one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK,
                                                      0xf, false));
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}

// Sum over the 64 lanes of a wavefront in a fixed order; the total lands in
// lane 63 (other lanes hold partial sums).
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
    v += dpp_f32<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141, 0xf>(v);  // row_half_mirror
    v += dpp_f32<0x140, 0xf>(v);  // row_mirror
    v += dpp_f32<0x142, 0xa>(v);  // row_bcast15 into rows 1 and 3
    v += dpp_f32<0x143, 0xc>(v);  // row_bcast31 into rows 2 and 3
    return v;
}

// The wave sums of NV per-lane values (NV = 8, 16 or 32) with the pairing of wave_sum_to_lane63 --
// lanes l^1, l^2, then quads, half rows, rows, halves; fp32 addition commutes, so the totals have
// the same bits -- as a transposing reduction: at each level a lane forms the pair sums of only half
// of the values it still holds and its partner those of the other half, so the work halves per
// level (NV + NV/2 + .. adds instead of 6 NV) and the NV totals end in NV different lanes.
// Which half a lane keeps at levels 1..4 is chosen so that the partner of the *next* levels
// (l^2, l^7, l^15: the DPP controls of the plain tree) holds the same values: bits
// b0^b2, b1^b2, b2^b3, b3 of the lane number; the row and half levels swap whole rows
// (v_permlane16_swap, v_permlane32_swap).  Returns the total of value wave_sum_transposed_index<NV>(lane);
// lanes 0..NV-1 cover every value once.
template <int NV>
__device__ __forceinline__ int wave_sum_transposed_index(int lane) {
    static_assert(NV == 8 || NV == 16 || NV == 32, "8, 16 or 32 values per lane");
    const int s1 = (lane ^ (lane >> 2)) & 1, s2 = ((lane >> 1) ^ (lane >> 2)) & 1;
    const int s3 = ((lane >> 2) ^ (lane >> 3)) & 1, s4 = (lane >> 3) & 1, s5 = (lane >> 4) & 1;
    if constexpr (NV == 8) return s1 * 4 + s2 * 2 + s3;
    else if constexpr (NV == 16) return s1 * 8 + s2 * 4 + s3 * 2 + s4;
    else return s1 * 16 + s2 * 8 + s3 * 4 + s4 * 2 + s5;
}

template <int CTRL, int H>
__device__ __forceinline__ void transposed_level(const float (&in)[2 * H], float (&out)[H], bool upper) {
#pragma unroll
    for (int i = 0; i < H; ++i) {
        const float lo = in[i] + dpp_f32<CTRL, 0xf>(in[i]);
        const float hi = in[i + H] + dpp_f32<CTRL, 0xf>(in[i + H]);
        out[i] = upper ? hi : lo;
    }
}

template <int NV>
__device__ __forceinline__ float wave_sum_transposed(const float (&v)[NV], int lane) {
    static_assert(NV == 8 || NV == 16 || NV == 32, "8, 16 or 32 values per lane");
    typedef unsigned u32x2_swap __attribute__((ext_vector_type(2)));
    float a1[NV / 2], a2[NV / 4], a3[NV / 8];
    transposed_level<0xB1, NV / 2>(v, a1, ((lane ^ (lane >> 2)) & 1) != 0);          // l ^ 1
    transposed_level<0x4E, NV / 4>(a1, a2, (((lane >> 1) ^ (lane >> 2)) & 1) != 0);  // l ^ 2
    transposed_level<0x141, NV / 8>(a2, a3, (((lane >> 2) ^ (lane >> 3)) & 1) != 0); // other quad of the half row
    float t;
    if constexpr (NV == 8) {
        t = a3[0] + dpp_f32<0x140, 0xf>(a3[0]);                                      // other half of the row
    } else {
        float a4[NV / 16];
        transposed_level<0x140, NV / 16>(a3, a4, ((lane >> 3) & 1) != 0);
        if constexpr (NV == 32) {
            // rows 0+1 and 2+3: even rows end with value 0, odd rows with value 1
            const u32x2_swap r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a4[0]), __float_as_uint(a4[1]), false, false);
            t = __uint_as_float(r.x) + __uint_as_float(r.y);
        } else {
            t = a4[0];
        }
    }
    if constexpr (NV != 32) {
        const u32x2_swap r = __builtin_amdgcn_permlane16_swap(__float_as_uint(t), __float_as_uint(t), false, false);
        t = __uint_as_float(r.x) + __uint_as_float(r.y);                              // rows 0+1, 2+3
    }
    const u32x2_swap h = __builtin_amdgcn_permlane32_swap(__float_as_uint(t), __float_as_uint(t), false, false);
    return __uint_as_float(h.x) + __uint_as_float(h.y);                               // the two halves
}

// Max over the 64 lanes; every lane of row 3 ends with the wave maximum, lane
// 63 included.  Inputs must be >= 0 (masked lanes contribute 0).
__device__ __forceinline__ float wave_max_to_lane63(float v) {
    v = fmaxf(v, dpp_f32<0xB1, 0xf>(v));
    v = fmaxf(v, dpp_f32<0x4E, 0xf>(v));
    v = fmaxf(v, dpp_f32<0x141, 0xf>(v));
    v = fmaxf(v, dpp_f32<0x140, 0xf>(v));
    v = fmaxf(v, dpp_f32<0x142, 0xa>(v));
    v = fmaxf(v, dpp_f32<0x143, 0xc>(v));
    return v;
}

// Workgroups are handed to the eight XCDs round-robin.  Renumbered so that each XCD works on one
// contiguous run of row blocks, the 2-byte results of neighbouring rows -- one cache line holds 64 of
// them -- are written by one XCD and leave its L2 as whole lines when the launch ends (lines whose
// bytes are spread over eight L2s cost the step of 129 decode launches 5 %).
__device__ __forceinline__ int xcd_contiguous_block(int b, int nb) {
    const int x = b & 7, q = nb >> 3, r = nb & 7;
    return x * q + min(x, r) + (b >> 3);
}

__device__ __forceinline__ float lane63(float v) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

}  // namespace cmi
