// Producers of quantised activations fused with the op in front of them:
//   silu_mul_quant   out = bf16(silu(gate)) * up (bf16), then the per-token int8 quantiser
//   rms_norm_i8      y = rms_norm(x) * w (bf16), then the quantiser
//   add_rms_norm_i8  x += add (bf16, written back), then the same
// Each equals "the op writing bf16, then cmi_quant_act_i8 reading it back" bit for bit: the
// absmax is taken over the narrowed bf16 values and the rounding is quant_math.hpp's.  What
// the fusion saves is the bf16 round trip through HBM in front of every W8A8 / W4A8
// projection (5 B per element instead of 9 for silu_mul_quant with the bf16 copy, 3 without).
//
// One workgroup per row; the row's results stay in registers across the absmax reduction
// (VPT 16-byte vectors per thread), so every input is read once and every output written once.
#include "quant_math.hpp"

namespace {

using namespace cmi;

constexpr int THREADS = 256;       // per row when there are rows enough to fill the chip
constexpr int MAX_THREADS = 1024;  // per row for a few rows: the row is the only parallelism there is
constexpr int FEW_ROWS = 256;      // up to this many rows a row gets as many threads as it has vectors

__device__ __forceinline__ float block_max(float v, float *smem) {
    v = wave_max_to_lane63(v);
    if ((threadIdx.x & 63) == 63) smem[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = smem[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) r = fmaxf(r, smem[i]);
    __syncthreads();  // smem is reused by the caller's next reduction
    return r;
}

// Sum of doubles over the workgroup.  The addends are sums of squares of bf16 values, which
// double holds exactly for any realistic row, so the order of this tree does not matter.
__device__ __forceinline__ double block_sum(double v, double *smem) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
    __syncthreads();
    double r = smem[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) r += smem[i];
    __syncthreads();
    return r;
}

// ----------------------------------------------------------------- silu

// silu(g) for a bf16 g as the fp32 value whose narrowing is the result: g / (1 + exp(-g))
// evaluated in fp32 with exp rounded once from its exact value.  The fast evaluation --
// exp(-g) = 2^p (1 + r ln 2) with p + r = -g log2(e) split exactly by an fma, v_exp_f32, v_rcp_f32 --
// is within 3 fp32 steps of that value for every bf16 g with |g| < 64 (measured over all of
// them); it is used unless it sits within 8 steps of a bf16 rounding boundary, where those few
// steps could change the narrowing: such inputs (0.02 %) and |g| >= 64, infinities and NaN take
// the double-precision exp and the correctly rounded division.
__device__ __forceinline__ float silu_exact_f32(float g) {
    const float e = (float)exp((double)(-g));
    return __fdiv_rn(g, 1.f + e);
}

__device__ __forceinline__ float silu_f32(float g) {
    if (!(fabsf(g) < 64.f)) return silu_exact_f32(g);
    constexpr float LOG2E = 1.44269502e+00f, LOG2E_LO = 1.92596299e-08f, LN2 = 0.693147182f;
    const float ng = -g;
    const float p = __fmul_rn(ng, LOG2E);
    const float r = __fadd_rn(__fmaf_rn(ng, LOG2E, -p), __fmul_rn(ng, LOG2E_LO));
    const float ep = __builtin_amdgcn_exp2f(p);
    const float e = __fmaf_rn(__fmul_rn(ep, LN2), r, ep);
    const float fast = __fmul_rn(g, __builtin_amdgcn_rcpf(__fadd_rn(1.f, e)));
    const uint32_t low = __float_as_uint(fast) & 0xffffu;
    if (low - (0x8000u - 8u) <= 16u) return silu_exact_f32(g);
    return fast;
}

__device__ __forceinline__ uint32_t silu_bf16_bits(float g) { return pack2_bf16(silu_f32(g), 0.f) & 0xffffu; }

// product of two bf16 values as torch forms it: one fp32 multiply, one narrowing
__device__ __forceinline__ uint32_t mul_bf16_bits(uint32_t a_bits, float b) {
    return pack2_bf16(__fmul_rn(bf16_bits_to_f32(a_bits), b), 0.f) & 0xffffu;
}

// eight elements: bf16(bf16(silu(g)) * u), two per dword
__device__ __forceinline__ uint4 silu_mul8(const uint4 &g, const uint4 &u) {
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t s2 = pack2_bf16(silu_f32(bf16_bits_to_f32(gw[i] & 0xffffu)),
                                       silu_f32(__uint_as_float(gw[i] & 0xffff0000u)));
        o[i] = pack2_bf16(__fmul_rn(bf16_bits_to_f32(s2 & 0xffffu), bf16_bits_to_f32(uw[i] & 0xffffu)),
                          __fmul_rn(__uint_as_float(s2 & 0xffff0000u), __uint_as_float(uw[i] & 0xffff0000u)));
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

struct SiluArgs {
    const uint16_t *gate, *up;
    uint16_t *out;   // nullable
    int8_t *q;       // nullable together with s
    float *s;
    int K;
    long ldg, ldu, ldo;
};

// K % 8 == 0, every row 16-byte aligned.  VPT > 0: the row fits VPT vectors per thread.
// T_MAX: the most threads a launch gives a row (blockDim.x is what it gives).
template <int VPT, int T_MAX = THREADS>
__global__ void __launch_bounds__(T_MAX) silu_mul_quant_vec(SiluArgs a) {
    __shared__ float smem[MAX_THREADS / 64];
    const int T = blockDim.x;
    const int row = blockIdx.x, nvec = a.K / 8;
    const uint4 *gr = reinterpret_cast<const uint4 *>(a.gate + (size_t)row * a.ldg);
    const uint4 *ur = reinterpret_cast<const uint4 *>(a.up + (size_t)row * a.ldu);
    uint4 *orow = a.out ? reinterpret_cast<uint4 *>(a.out + (size_t)row * a.ldo) : nullptr;
    uint4 v[VPT];
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int idx = threadIdx.x + i * T;
        if (idx < nvec) {
            v[i] = silu_mul8(gr[idx], ur[idx]);
            if (orow) orow[idx] = v[i];  // may overwrite up[idx]: read above by this same thread
        } else {
            v[i] = make_uint4(0, 0, 0, 0);
        }
    }
    if (!a.q) return;
#pragma unroll
    for (int i = 0; i < VPT; ++i) amax = absmax8(v[i], amax);
    amax = block_max(amax, smem);
    const RowScale rs = row_scale(amax);
    if (threadIdx.x == 0) a.s[row] = rs.sc;
    uint2 *qr = reinterpret_cast<uint2 *>(a.q + (size_t)row * a.K);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int idx = threadIdx.x + i * T;
        if (idx < nvec) qr[idx] = quant8(v[i], rs);
    }
}

// Any K, pitch and alignment; rows longer than the vector kernel holds.  Two passes: the
// product is recomputed for the quantiser (cheaper than depending on a bf16 copy that the
// caller may not have asked for).
__global__ void __launch_bounds__(THREADS) silu_mul_quant_scalar(SiluArgs a) {
    __shared__ float smem[MAX_THREADS / 64];
    const int row = blockIdx.x;
    const uint16_t *gr = a.gate + (size_t)row * a.ldg, *ur = a.up + (size_t)row * a.ldu;
    int8_t *qr = a.q ? a.q + (size_t)row * a.K : nullptr;
    // the quantised row must come from the inputs as they were: quantise before `out` (which may
    // alias `up`) is written
    float amax = 0.f;
    if (a.q) {
        for (int k = threadIdx.x; k < a.K; k += THREADS) {
            const uint32_t p = mul_bf16_bits(silu_bf16_bits(bf16_bits_to_f32(gr[k])), bf16_bits_to_f32(ur[k]));
            amax = fmaxf(amax, fabsf(bf16_bits_to_f32(p)));
        }
        amax = block_max(amax, smem);
    }
    const RowScale rs = row_scale(amax);
    if (a.q && threadIdx.x == 0) a.s[row] = rs.sc;
    uint16_t *orow = a.out ? a.out + (size_t)row * a.ldo : nullptr;
    for (int k = threadIdx.x; k < a.K; k += THREADS) {
        const uint32_t p = mul_bf16_bits(silu_bf16_bits(bf16_bits_to_f32(gr[k])), bf16_bits_to_f32(ur[k]));
        if (qr) qr[k] = (int8_t)quant1(bf16_bits_to_f32(p), rs);
        if (orow) orow[k] = (uint16_t)p;
    }
}

// ------------------------------------------------------------- rms norm

struct NormArgs {
    uint16_t *x;          // read; written back when add != nullptr
    const uint16_t *add;  // nullable
    const uint16_t *w;
    uint16_t *y;          // nullable: the bf16 normalised row
    int8_t *q;            // nullable together with s
    float *s;
    int N;
    long ldx, lda, ldy;
    float eps;
};

__device__ __forceinline__ float inv_rms(double ss, int N, float eps) {
    const float ms = (float)(ss / (double)N);
    return __fdiv_rn(1.0f, __fsqrt_rn(ms + eps));
}

__device__ __forceinline__ uint32_t add_bf16_bits(float a, float b) { return pack2_bf16(__fadd_rn(a, b), 0.f) & 0xffffu; }

__device__ __forceinline__ uint32_t norm1(float x, float scale, float w) {
    return mul_bf16_bits(pack2_bf16(__fmul_rn(x, scale), 0.f) & 0xffffu, w);
}

// the two bf16 of a dword at once: bf16(bf16(x * scale) * w)
__device__ __forceinline__ uint32_t norm2(uint32_t xw, float scale, uint32_t gw) {
    const uint32_t t = pack2_bf16(__fmul_rn(bf16_bits_to_f32(xw & 0xffffu), scale),
                                  __fmul_rn(__uint_as_float(xw & 0xffff0000u), scale));
    return pack2_bf16(__fmul_rn(bf16_bits_to_f32(t & 0xffffu), bf16_bits_to_f32(gw & 0xffffu)),
                      __fmul_rn(__uint_as_float(t & 0xffff0000u), __uint_as_float(gw & 0xffff0000u)));
}

__device__ __forceinline__ uint32_t add2(uint32_t xw, uint32_t dw) {
    return pack2_bf16(__fadd_rn(bf16_bits_to_f32(xw & 0xffffu), bf16_bits_to_f32(dw & 0xffffu)),
                      __fadd_rn(__uint_as_float(xw & 0xffff0000u), __uint_as_float(dw & 0xffff0000u)));
}

template <int VPT, int T_MAX = THREADS>
__global__ void __launch_bounds__(T_MAX) rms_norm_i8_vec(NormArgs a) {
    __shared__ double dsmem[MAX_THREADS / 64];
    __shared__ float smem[MAX_THREADS / 64];
    const int T = blockDim.x;
    const int row = blockIdx.x, nvec = a.N / 8;
    uint4 *xr = reinterpret_cast<uint4 *>(a.x + (size_t)row * a.ldx);
    const uint4 *ar = a.add ? reinterpret_cast<const uint4 *>(a.add + (size_t)row * a.lda) : nullptr;
    const uint4 *wr = reinterpret_cast<const uint4 *>(a.w);
    uint4 v[VPT];
    double ss = 0.0;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int idx = threadIdx.x + i * T;
        if (idx < nvec) {
            v[i] = xr[idx];
            if (ar) {
                const uint4 d = ar[idx];
                const uint32_t xw[4] = {v[i].x, v[i].y, v[i].z, v[i].w}, dw[4] = {d.x, d.y, d.z, d.w};
                uint32_t o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = add2(xw[j], dw[j]);
                v[i] = make_uint4(o[0], o[1], o[2], o[3]);
                xr[idx] = v[i];  // the residual stream keeps the sum
            }
            const uint32_t w4[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const double lo = (double)bf16_bits_to_f32(w4[j] & 0xffffu);
                const double hi = (double)__uint_as_float(w4[j] & 0xffff0000u);
                ss = fma(lo, lo, ss);
                ss = fma(hi, hi, ss);
            }
        } else {
            v[i] = make_uint4(0, 0, 0, 0);
        }
    }
    const float scale = inv_rms(block_sum(ss, dsmem), a.N, a.eps);
    uint4 *yr = a.y ? reinterpret_cast<uint4 *>(a.y + (size_t)row * a.ldy) : nullptr;
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int idx = threadIdx.x + i * T;
        if (idx < nvec) {
            const uint4 g = wr[idx];
            const uint32_t xw[4] = {v[i].x, v[i].y, v[i].z, v[i].w}, gw[4] = {g.x, g.y, g.z, g.w};
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = norm2(xw[j], scale, gw[j]);
            v[i] = make_uint4(o[0], o[1], o[2], o[3]);
            if (yr) yr[idx] = v[i];
            amax = absmax8(v[i], amax);
        }
    }
    if (!a.q) return;
    amax = block_max(amax, smem);
    const RowScale rs = row_scale(amax);
    if (threadIdx.x == 0) a.s[row] = rs.sc;
    uint2 *qr = reinterpret_cast<uint2 *>(a.q + (size_t)row * a.N);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int idx = threadIdx.x + i * T;
        if (idx < nvec) qr[idx] = quant8(v[i], rs);
    }
}

// Short rows (N <= 4096): one wavefront per row, VPT vectors per lane.  The sum of squares and
// the absmax are reduced inside the wavefront, so a row costs no LDS and no barrier -- with one
// workgroup per 5 KB row the three barriers were most of the row's latency (8192 x 2560:
// 22 -> 13 us).  Same arithmetic, same bits.
template <int VPT>
__global__ void __launch_bounds__(THREADS) rms_norm_i8_wave(NormArgs a, int rows) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (THREADS / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;  // whole wavefronts: nothing below synchronises across them
    const int nvec = a.N / 8;
    uint4 *xr = reinterpret_cast<uint4 *>(a.x + (size_t)row * a.ldx);
    const uint4 *ar = a.add ? reinterpret_cast<const uint4 *>(a.add + (size_t)row * a.lda) : nullptr;
    const uint4 *wr = reinterpret_cast<const uint4 *>(a.w);
    uint4 v[VPT];
    double ss = 0.0;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int idx = lane + i * 64;
        if (idx < nvec) {
            v[i] = xr[idx];
            if (ar) {
                const uint4 d = ar[idx];
                v[i] = make_uint4(add2(v[i].x, d.x), add2(v[i].y, d.y), add2(v[i].z, d.z), add2(v[i].w, d.w));
                xr[idx] = v[i];  // the residual stream keeps the sum
            }
            const uint32_t w4[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const double lo = (double)bf16_bits_to_f32(w4[j] & 0xffffu);
                const double hi = (double)__uint_as_float(w4[j] & 0xffff0000u);
                ss = fma(lo, lo, ss);
                ss = fma(hi, hi, ss);
            }
        } else {
            v[i] = make_uint4(0, 0, 0, 0);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);  // exact addends: any order
    const float scale = inv_rms(ss, a.N, a.eps);
    uint4 *yr = a.y ? reinterpret_cast<uint4 *>(a.y + (size_t)row * a.ldy) : nullptr;
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int idx = lane + i * 64;
        if (idx < nvec) {
            const uint4 g = wr[idx];
            v[i] = make_uint4(norm2(v[i].x, scale, g.x), norm2(v[i].y, scale, g.y), norm2(v[i].z, scale, g.z),
                              norm2(v[i].w, scale, g.w));
            if (yr) yr[idx] = v[i];
            amax = absmax8(v[i], amax);
        }
    }
    if (!a.q) return;
    amax = lane63(wave_max_to_lane63(amax));
    const RowScale rs = row_scale(amax);
    if (lane == 0) a.s[row] = rs.sc;
    uint2 *qr = reinterpret_cast<uint2 *>(a.q + (size_t)row * a.N);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int idx = lane + i * 64;
        if (idx < nvec) qr[idx] = quant8(v[i], rs);
    }
}

// Any N, pitch and alignment.  Needs a bf16 destination for the normalised row when quantising
// (y, or the quantiser would have to recompute it a third time): the host passes one.
__global__ void __launch_bounds__(THREADS) rms_norm_i8_scalar(NormArgs a) {
    __shared__ double dsmem[MAX_THREADS / 64];
    __shared__ float smem[MAX_THREADS / 64];
    const int row = blockIdx.x;
    uint16_t *xr = a.x + (size_t)row * a.ldx;
    const uint16_t *ar = a.add ? a.add + (size_t)row * a.lda : nullptr;
    double ss = 0.0;
    for (int k = threadIdx.x; k < a.N; k += THREADS) {
        uint32_t b = xr[k];
        if (ar) {
            b = add_bf16_bits(bf16_bits_to_f32(b), bf16_bits_to_f32(ar[k]));
            xr[k] = (uint16_t)b;
        }
        const double v = (double)bf16_bits_to_f32(b);
        ss = fma(v, v, ss);
    }
    const float scale = inv_rms(block_sum(ss, dsmem), a.N, a.eps);
    float amax = 0.f;
    for (int k = threadIdx.x; k < a.N; k += THREADS)   // xr[k] was written by this same thread
        amax = fmaxf(amax, fabsf(bf16_bits_to_f32(norm1(bf16_bits_to_f32(xr[k]), scale, bf16_bits_to_f32(a.w[k])))));
    amax = block_max(amax, smem);
    const RowScale rs = row_scale(amax);
    if (a.q && threadIdx.x == 0) a.s[row] = rs.sc;
    uint16_t *yr = a.y ? a.y + (size_t)row * a.ldy : nullptr;
    int8_t *qr = a.q ? a.q + (size_t)row * a.N : nullptr;
    for (int k = threadIdx.x; k < a.N; k += THREADS) {
        const uint32_t p = norm1(bf16_bits_to_f32(xr[k]), scale, bf16_bits_to_f32(a.w[k]));
        if (yr) yr[k] = (uint16_t)p;
        if (qr) qr[k] = (int8_t)quant1(bf16_bits_to_f32(p), rs);
    }
}

template <typename Args, typename K1, typename K2, typename K4, typename K8, typename K16>
void launch_vpt(int vpt, const Args &a, int rows, hipStream_t st, K1 k1, K2 k2, K4 k4, K8 k8, K16 k16) {
    const dim3 grid(rows), block(THREADS);
    if (vpt <= 1) k1<<<grid, block, 0, st>>>(a);
    else if (vpt <= 2) k2<<<grid, block, 0, st>>>(a);
    else if (vpt <= 4) k4<<<grid, block, 0, st>>>(a);
    else if (vpt <= 8) k8<<<grid, block, 0, st>>>(a);
    else k16<<<grid, block, 0, st>>>(a);
}

int norm_entry(const char *who, uint16_t *x, const uint16_t *add, const void *w, void *y, int8_t *q, float *s,
               int M, int N, long ldx, long lda, long ldy, float eps, void *stream) {
    CMI_REQUIRE(M >= 0 && N > 0, CMI_E_ARG, "%s: bad shape M=%d N=%d", who, M, N);
    if (M == 0) return CMI_OK;
    CMI_REQUIRE(x && w && ((q && s) || y), CMI_E_ARG, "%s: null pointer (x, w and one of y or out_q + out_s)", who);
    CMI_REQUIRE((q == nullptr) == (s == nullptr), CMI_E_ARG, "%s: out_q and out_s go together", who);
    CMI_REQUIRE(ldx >= N && (!add || lda >= N) && (!y || ldy >= N), CMI_E_ARG, "%s: a row pitch is below N=%d", who, N);
    CMI_REQUIRE(eps >= 0.f, CMI_E_ARG, "%s: eps must not be negative", who);
    NormArgs a{x, add, static_cast<const uint16_t *>(w), static_cast<uint16_t *>(y), q, s, N, ldx, lda, ldy, eps};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int nvec = N / 8, vpt = (nvec + THREADS - 1) / THREADS;
    const bool vec = N % 8 == 0 && vpt <= 16 && aligned(x, 16) && ldx % 8 == 0 && aligned(w, 16) &&
                     (!add || (aligned(add, 16) && lda % 8 == 0)) && (!y || (aligned(y, 16) && ldy % 8 == 0)) &&
                     (!q || aligned(q, 8));
    if (vec && M <= FEW_ROWS && nvec <= 2 * MAX_THREADS) {
        // a few rows: latency, not throughput -- every vector of the row gets a thread of its own
        const int t = nvec <= MAX_THREADS ? (nvec + 63) / 64 * 64 : MAX_THREADS;
        if (nvec <= MAX_THREADS) rms_norm_i8_vec<1, MAX_THREADS><<<dim3(M), dim3(t), 0, st>>>(a);
        else rms_norm_i8_vec<2, MAX_THREADS><<<dim3(M), dim3(t), 0, st>>>(a);
    } else if (vec && nvec <= 8 * 64) {
        const dim3 grid((M + THREADS / 64 - 1) / (THREADS / 64)), block(THREADS);
        const int wvpt = (nvec + 63) / 64;
        if (wvpt <= 1) rms_norm_i8_wave<1><<<grid, block, 0, st>>>(a, M);
        else if (wvpt <= 2) rms_norm_i8_wave<2><<<grid, block, 0, st>>>(a, M);
        else if (wvpt <= 3) rms_norm_i8_wave<3><<<grid, block, 0, st>>>(a, M);
        else if (wvpt <= 4) rms_norm_i8_wave<4><<<grid, block, 0, st>>>(a, M);
        else if (wvpt <= 5) rms_norm_i8_wave<5><<<grid, block, 0, st>>>(a, M);
        else if (wvpt <= 6) rms_norm_i8_wave<6><<<grid, block, 0, st>>>(a, M);
        else rms_norm_i8_wave<8><<<grid, block, 0, st>>>(a, M);
    } else if (vec)
        launch_vpt(vpt, a, M, st, rms_norm_i8_vec<1>, rms_norm_i8_vec<2>, rms_norm_i8_vec<4>, rms_norm_i8_vec<8>,
                   rms_norm_i8_vec<16>);
    else
        rms_norm_i8_scalar<<<dim3(M), dim3(THREADS), 0, st>>>(a);
    return check_launch(who);
}

}  // namespace

extern "C" int cmi_silu_mul_quant(const void *gate, const void *up, void *out, int8_t *out_q, float *out_s,
                                  int M, int K, int64_t ld_gate, int64_t ld_up, int64_t ld_out, void *stream) {
    CMI_REQUIRE(M >= 0 && K > 0, CMI_E_ARG, "cmi_silu_mul_quant: bad shape M=%d K=%d", M, K);
    if (M == 0) return CMI_OK;
    CMI_REQUIRE(gate && up && (out || (out_q && out_s)), CMI_E_ARG,
                "cmi_silu_mul_quant: null pointer (gate, up and one of out or out_q + out_s)");
    CMI_REQUIRE((out_q == nullptr) == (out_s == nullptr), CMI_E_ARG, "cmi_silu_mul_quant: out_q and out_s go together");
    CMI_REQUIRE(ld_gate >= K && ld_up >= K && (!out || ld_out >= K), CMI_E_ARG,
                "cmi_silu_mul_quant: a row pitch is below K=%d", K);
    SiluArgs a{static_cast<const uint16_t *>(gate), static_cast<const uint16_t *>(up), static_cast<uint16_t *>(out),
               out_q, out_s, K, (long)ld_gate, (long)ld_up, (long)ld_out};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int nvec = K / 8, vpt = (nvec + THREADS - 1) / THREADS;
    const bool vec = K % 8 == 0 && vpt <= 16 && aligned(gate, 16) && aligned(up, 16) && ld_gate % 8 == 0 &&
                     ld_up % 8 == 0 && (!out || (aligned(out, 16) && ld_out % 8 == 0)) && (!out_q || aligned(out_q, 8));
    if (vec && M <= FEW_ROWS && nvec <= 2 * MAX_THREADS) {
        // a few rows: latency, not throughput -- every vector of the row gets a thread of its own
        const int t = nvec <= MAX_THREADS ? (nvec + 63) / 64 * 64 : MAX_THREADS;
        if (nvec <= MAX_THREADS) silu_mul_quant_vec<1, MAX_THREADS><<<dim3(M), dim3(t), 0, st>>>(a);
        else silu_mul_quant_vec<2, MAX_THREADS><<<dim3(M), dim3(t), 0, st>>>(a);
    } else if (vec)
        launch_vpt(vpt, a, M, st, silu_mul_quant_vec<1>, silu_mul_quant_vec<2>, silu_mul_quant_vec<4>,
                   silu_mul_quant_vec<8>, silu_mul_quant_vec<16>);
    else
        silu_mul_quant_scalar<<<dim3(M), dim3(THREADS), 0, st>>>(a);
    return check_launch("cmi_silu_mul_quant");
}

extern "C" int cmi_rms_norm_i8(const void *x, const void *w, void *y, int8_t *out_q, float *out_s, int M, int N,
                               int64_t ld_x, int64_t ld_y, float eps, void *stream) {
    return norm_entry("cmi_rms_norm_i8", const_cast<uint16_t *>(static_cast<const uint16_t *>(x)), nullptr, w, y,
                      out_q, out_s, M, N, (long)ld_x, 0, (long)ld_y, eps, stream);
}

extern "C" int cmi_add_rms_norm_i8(void *x, const void *add, const void *w, void *y, int8_t *out_q, float *out_s,
                                   int M, int N, int64_t ld_x, int64_t ld_add, int64_t ld_y, float eps, void *stream) {
    CMI_REQUIRE(add, CMI_E_ARG, "cmi_add_rms_norm_i8: null pointer (add)");
    return norm_entry("cmi_add_rms_norm_i8", static_cast<uint16_t *>(x), static_cast<const uint16_t *>(add), w, y,
                      out_q, out_s, M, N, (long)ld_x, (long)ld_add, (long)ld_y, eps, stream);
}
