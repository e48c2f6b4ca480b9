// int4 weight-only GEMV (W4A16): group-quantised int4 weights against *unquantised* bf16
// activations, one activation row -- the arithmetic the reference's torch path gives an int4
// weight (dequantise, then a floating-point product; backends/reference/__init__.py:93-95 with
// w4a8_weights.py:96-99) and the job of its gemv_kn_w4 (backends/corex/kernels/gemv.cu:1918-1930):
//
//   y[n] = bf16( sum_g ws[n,g] * sum_{k in g} (code(n,k) - 8) * x[k] ),   fp32 sums
//
// HBM-bound on the packed weight (half a byte per element), on the device layout of
// cmi_w4_repack.  One wavefront per weight row; a lane's 16-byte load is 32 codes of one group
// (four adjacent lanes own a group of 128).  Codes become bf16 without a conversion: 0x4300 | c
// is 128 + c exactly, two per dword after one byte permute, and go straight into
// v_dot2_f32_bf16 against the packed activations; the bias is taken out per group,
//   sum (c - 8) x = sum (128 + c) x - 136 * sum x,
// with the group sums of x formed once per workgroup.  Summation order (a function of K only):
// a lane chains its 32 products in k order from 0.f, the four lanes of a group are added by two
// quad permutes, a quad accumulates scale * group over its passes (ascending k) with one fma per
// group, and the 16 quads are added by the fixed wavefront tree.
#include "common.hpp"

namespace {

using namespace cmi;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GS = 128;
constexpr int WAVES = 4;
constexpr int MAX_PASSES = 16;
constexpr int MAX_K = MAX_PASSES * 2048;  // a wavefront keeps its whole row in registers: 4 per pass

struct Args {
    const uint8_t *w4;
    const float *ws;
    const uint16_t *x;
    uint16_t *y;
    int N, K, G;
};

__device__ __forceinline__ float dot_chunk(const u32x4 &w, const uint4 (&xv)[4]) {
    const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t lo = ww[i] & 0x0F0F0F0Fu, hi = (ww[i] >> 4) & 0x0F0F0F0Fu;
        // bytes -> 16-bit lanes, then 128 + code as bf16
        const uint32_t p0 = __builtin_amdgcn_perm(0u, lo, 0x0c010c00u) | 0x43004300u;
        const uint32_t p1 = __builtin_amdgcn_perm(0u, lo, 0x0c030c02u) | 0x43004300u;
        const uint32_t p2 = __builtin_amdgcn_perm(0u, hi, 0x0c010c00u) | 0x43004300u;
        const uint32_t p3 = __builtin_amdgcn_perm(0u, hi, 0x0c030c02u) | 0x43004300u;
        const uint32_t xd[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w};  // k = 8i .. 8i+7, two per dword
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p0), __builtin_bit_cast(bf16x2_t, xd[0]), acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p1), __builtin_bit_cast(bf16x2_t, xd[1]), acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p2), __builtin_bit_cast(bf16x2_t, xd[2]), acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p3), __builtin_bit_cast(bf16x2_t, xd[3]), acc, false);
    }
    return acc;
}

// NP: passes of 64 chunks (2048 k) a wavefront makes over its row.
template <int NP>
__global__ void __launch_bounds__(64 * WAVES)
gemv_w4a16_kernel(const Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint4 *xlds = reinterpret_cast<uint4 *>(lds);                       // bf16 [K]
    float *xsum = reinterpret_cast<float *>(lds + (size_t)a.K * 2);     // fp32 [G]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_raw = xcd_contiguous_block(blockIdx.x, gridDim.x) * WAVES + wave;
    const int n = n_raw < a.N ? n_raw : a.N - 1;
    const int nchunks = a.K / 32, xvecs = a.K / 8;

    // activations first (memory answers in request order), then every weight byte of the row
    constexpr int XV = NP;  // NP * 2048 k / 8 per vector / 256 threads
    uint4 xstage[XV];
    const uint4 *xg = reinterpret_cast<const uint4 *>(a.x);
#pragma unroll
    for (int j = 0; j < XV; ++j) {
        const int idx = threadIdx.x + j * 64 * WAVES;
        xstage[j] = idx < xvecs ? xg[idx] : make_uint4(0, 0, 0, 0);
    }
    const u32x4 *wrow = reinterpret_cast<const u32x4 *>(a.w4 + (size_t)n * (a.K / 2));
    u32x4 w[NP];
    float sc[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int c = p * 64 + lane;
        w[p] = __builtin_nontemporal_load(wrow + min(c, nchunks - 1));
        sc[p] = a.ws[(size_t)n * a.G + min(c >> 2, a.G - 1)];
    }
#pragma unroll
    for (int j = 0; j < XV; ++j) {
        const int idx = threadIdx.x + j * 64 * WAVES;
        if (idx < xvecs) xlds[idx] = xstage[j];
    }
    __syncthreads();
    // group sums of x: thread t takes chunk t (32 elements, k order), quads add up
    for (int c0 = 0; c0 < nchunks; c0 += 64 * WAVES) {
        const int c = c0 + threadIdx.x;
        const int cs = c < nchunks ? c : nchunks - 1;
        float s = 0.f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const uint4 q = xlds[cs * 4 + v];
            const uint32_t d[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s += bf16_bits_to_f32(d[i] & 0xffffu);
                s += __uint_as_float(d[i] & 0xffff0000u);
            }
        }
        s += dpp_f32<0xB1, 0xf>(s);
        s += dpp_f32<0x4E, 0xf>(s);
        if (c < nchunks && (threadIdx.x & 3) == 0) xsum[c >> 2] = s;
    }
    __syncthreads();

    float total = 0.f;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int c = p * 64 + lane;
        const bool live = c < nchunks;
        const int cs = live ? c : nchunks - 1;
        uint4 xv[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) xv[v] = xlds[cs * 4 + v];
        float d = dot_chunk(w[p], xv);
        d += dpp_f32<0xB1, 0xf>(d);
        d += dpp_f32<0x4E, 0xf>(d);
        const float t = __fmaf_rn(-136.f, xsum[cs >> 2], d);
        total = live ? __fmaf_rn(sc[p], t, total) : total;
    }
    // the four lanes of a quad hold the same value: one of them enters the wavefront sum
    total = (lane & 3) == 0 ? total : 0.f;
    total = wave_sum_to_lane63(total);
    if (lane == 63 && n_raw < a.N) a.y[n] = (uint16_t)f32_to_bf16_bits(total);
}

template <int NP>
int launch(const Args &a, hipStream_t st) {
    const size_t lds = (size_t)a.K * 2 + sizeof(float) * a.G;
    if (NP * 2048 * 2 > 60 * 1024) {  // beyond what a launch may ask for without saying so first
        static std::atomic<uint64_t> devices{0};
        if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemv_w4a16_kernel<NP>),
                                       NP * 2048 * 2 + (int)sizeof(float) * (NP * 2048 / GS), devices, "cmi_gemv_w4a16"))
            return rc;
    }
    gemv_w4a16_kernel<NP><<<dim3((a.N + WAVES - 1) / WAVES), dim3(64 * WAVES), lds, st>>>(a);
    return check_launch("cmi_gemv_w4a16");
}

}  // namespace

extern "C" int cmi_gemv_w4a16(const uint8_t *w4, const float *ws, const void *x, void *y, int N, int K, int gs,
                              void *stream) {
    CMI_REQUIRE(w4 && ws && x && y, CMI_E_ARG, "cmi_gemv_w4a16: null pointer");
    CMI_REQUIRE(N >= 1 && K >= GS, CMI_E_ARG, "cmi_gemv_w4a16: bad shape N=%d K=%d", N, K);
    CMI_REQUIRE(gs == GS && K % GS == 0, CMI_E_UNSUPPORTED,
                "cmi_gemv_w4a16: group size %d, K=%d; built for group size %d and K a multiple of it", gs, K, GS);
    CMI_REQUIRE(K <= MAX_K, CMI_E_UNSUPPORTED, "cmi_gemv_w4a16: K=%d above %d", K, MAX_K);
    CMI_REQUIRE(aligned(w4, 16) && aligned(x, 16) && aligned(ws, 4) && aligned(y, 2), CMI_E_ARG,
                "cmi_gemv_w4a16: w4 and x must be 16-byte aligned");
    Args a{w4, ws, static_cast<const uint16_t *>(x), static_cast<uint16_t *>(y), N, K, K / GS};
    hipStream_t st = static_cast<hipStream_t>(stream);
    // one instantiation per pass count up to 5 (K <= 10240: the decode shapes), then steps of 2 and 3
    const int passes = (K / 32 + 63) / 64;
    switch (passes) {
        case 1: return launch<1>(a, st);
        case 2: return launch<2>(a, st);
        case 3: return launch<3>(a, st);
        case 4: return launch<4>(a, st);
        case 5: return launch<5>(a, st);
        case 6:
        case 7: return launch<7>(a, st);
        case 8:
        case 9: return launch<9>(a, st);
        case 10:
        case 11: return launch<11>(a, st);
        case 12:
        case 13: return launch<13>(a, st);
        default: return launch<16>(a, st);
    }
}
