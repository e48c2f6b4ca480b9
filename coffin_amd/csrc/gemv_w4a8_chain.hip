// W4A8 decode GEMV with the fp32 chain kept in registers: bf16 or already quantised activations,
// one or two rows, every wavefront requesting all of its weight bytes up front (K <= 5120 per
// wavefront; longer rows, up to 20480, are shared by two to eight wavefronts).
//
//   xq, xs  = per-token int8 quantisation of x (arithmetic of cmi_quant_act_i8)
//   sum_g   = sum_{k in group g} xq[m,k] * (code(n,k) - 8)     int32, exact
//   total   = fma((float)sum_g, ws[n,g], total)                 g = 0,1,.. from 0.f
//   y[m,n]  = bf16(total * xs[m])
//
// Same arithmetic and bits as gemv_w4a8_decode_kernel; what differs is where the instructions go.
//
// * No unpacking of the codes.  The workgroup stores the activations as two planes of unsigned
//   nibbles, x + 128 = 16 a + b, arranged in the nibble order of the weight words, and
//   v_dot8_u32_u4 multiplies eight codes with eight nibbles:
//       sum (c - 8) x = 16 (sum c a - 8 sum c) + (sum c b - 8 sum x)
//   -- three dot instructions per weight word (the third, against 0x88888888, is 8 sum c) instead
//   of three mask/shift instructions and two v_dot4; -8 sum x per 32-element chunk is the start
//   value of the b accumulator, formed once per workgroup.
// * LPR lanes own one weight row (128 or 256 contiguous bytes per load instruction), so the four
//   lanes of a group are a DPP quad and a load instruction covers LPR/4 whole groups of 64/LPR
//   rows.  After two quad permutes every lane of a quad holds its group's integer sum; the first
//   quad of the row converts it and extends the row's fp32 chain, fetching the sums of the row's
//   other quads with row shifts.  Loads are consumed in k order, so the chain sees the groups
//   in order: no parking of partial sums in LDS, no serial walk at the end, no second barrier.
//   Groups past K meet a scale of 0.f: fma(finite, 0, total) is total (the chain starts at +0
//   and cannot reach -0).
// * Longer rows are shared by S wavefronts of a workgroup, each a contiguous run of loads: every
//   wavefront forms and converts its integer sums as its bytes arrive, then the chain passes
//   through the S wavefronts in k order, its running value handed over in LDS (S - 1 barriers).
#include "quant_math.hpp"

namespace {

using namespace cmi;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GS = 128;

struct Args {
    const uint8_t *w4;
    const float *ws;
    const uint16_t *x;   // bf16 activations (PREQ == false)
    const int8_t *xq;    // quantised activations and their scales (PREQ == true)
    const float *xs;
    uint16_t *y;
    int32_t *group_acc;
    int8_t *xq_out;
    float *xs_out;
    int M, N, K, G;
};

// Two words of x + 128 (bytes k0..k0+3 and k0+4..k0+7) -> their high-nibble and low-nibble words in
// the order of a weight word: nibble 2b belongs to k0 + b, nibble 2b + 1 to k0 + 4 + b.
__device__ __forceinline__ void nibble_planes(uint32_t u0, uint32_t u1, uint32_t &hi, uint32_t &lo) {
    hi = ((u0 >> 4) & 0x0F0F0F0Fu) | (u1 & 0xF0F0F0F0u);
    lo = (u0 & 0x0F0F0F0Fu) | ((u1 << 4) & 0xF0F0F0F0u);
}

// LDS: per activation row CP chunk slots of 32 bytes (high-nibble words, then low-nibble words, of 32
// elements), then CP start values (-8 * sum of the chunk), then the row scales and the partial maxima.
template <int M, int CP, int WAVES>
struct Lds {
    static constexpr int planes = 0;
    static constexpr int xsum = planes + M * CP * 32;
    static constexpr int xs = xsum + M * CP * 4;
    static constexpr int part = xs + 16;                // float [M][WAVES]: partial maxima
    static constexpr int carry = part + 4 * M * WAVES;  // float [WAVES][M][16]: the chain between wavefronts
    static constexpr int total = carry + 4 * WAVES * M * 16;
};

// M: activation rows (1, 2).  LPR: lanes per weight row (8, 16).  NL: load instructions per wavefront,
// each covering LPR * 32 elements of every row.  PREQ: activations arrive quantised.
// EXACT: K == S * NL * LPR * 32 and the integer sums are not asked for -- no clamped addresses, no
// scale selects, no early exit from the loads.  S: wavefronts that share the same rows, each taking
// NL consecutive loads.  WAVES: wavefronts per workgroup (WAVES / S teams).
template <int M, int LPR, int NL, bool PREQ, bool EXACT, int S, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
gemv_w4a8_chain_kernel(const Args a) {
    constexpr int THREADS = 64 * WAVES;
    constexpr int RPW = 64 / LPR, Q = LPR / 4, CP = S * NL * LPR;
    using L = Lds<M, CP, WAVES>;
    extern __shared__ __align__(16) uint8_t lds[];
    uint4 *planes = reinterpret_cast<uint4 *>(lds + L::planes);
    int32_t *xsum = reinterpret_cast<int32_t *>(lds + L::xsum);
    float *xs_lds = reinterpret_cast<float *>(lds + L::xs);
    float *part = reinterpret_cast<float *>(lds + L::part);
    float *carry = reinterpret_cast<float *>(lds + L::carry);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane % LPR, r = lane / LPR;
    const int team = wave / S, part_s = wave % S;  // which rows, which run of loads
    const int j0 = part_s * NL;                     // first load of this wavefront
    const int block = xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int n_raw = (block * (WAVES / S) + team) * RPW + r;
    const int n = min(n_raw, a.N - 1);
    const int nchunks = a.K / 32;

    // 1. activations first (memory answers in request order and they are needed first)
    constexpr int XVN = PREQ ? (CP * 2 + THREADS - 1) / THREADS : (CP * 4 + THREADS - 1) / THREADS;
    const int xvecs = PREQ ? a.K / 16 : a.K / 8;
    uint4 v[M][XVN];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int mrow = m < a.M ? m : a.M - 1;
        const uint4 *xg = PREQ ? reinterpret_cast<const uint4 *>(a.xq + (size_t)mrow * a.K)
                               : reinterpret_cast<const uint4 *>(a.x + (size_t)mrow * a.K);
#pragma unroll
        for (int j = 0; j < XVN; ++j) {
            const int idx = threadIdx.x + j * THREADS;
            v[m][j] = idx < xvecs ? xg[idx] : make_uint4(0, 0, 0, 0);
        }
    }
    // 2. every weight byte of this wavefront's rows, and behind each load the group scales that its
    // sums will meet (memory answers in request order: the chain can start with the first load).
    // 0.f past K.
    const u32x4 *wrow = reinterpret_cast<const u32x4 *>(a.w4 + (size_t)n * (a.K / 2));
    const float *wsrow = a.ws + (size_t)n * a.G;
    u32x4 w[NL];
    float wsr[NL][Q];
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        w[j] = __builtin_nontemporal_load(wrow + (EXACT ? (j0 + j) * LPR + c : min((j0 + j) * LPR + c, nchunks - 1)));
        if constexpr (EXACT) {
            typedef float fq_t __attribute__((ext_vector_type(Q)));
            fq_t t;
            __builtin_memcpy(&t, wsrow + (j0 + j) * Q, sizeof(t));
#pragma unroll
            for (int q = 0; q < Q; ++q) wsr[j][q] = t[q];
        } else {
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int g = (j0 + j) * Q + q;  // uniform
                const float sc = wsrow[min(g, a.G - 1)];
                wsr[j][q] = g < a.G ? sc : 0.f;
            }
        }
    }

    // 4. nibble planes of x + 128 and the chunk start values, into LDS
    if constexpr (PREQ) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            if (threadIdx.x == 0) xs_lds[m] = a.xs[m < a.M ? m : a.M - 1];
#pragma unroll
            for (int j = 0; j < XVN; ++j) {
                if (j * THREADS >= xvecs) break;  // uniform
                const int idx = threadIdx.x + j * THREADS;  // 16 elements: half a chunk
                const uint4 q = v[m][j];
                int s8 = __builtin_amdgcn_sdot4((int)q.x, 0x01010101, 0, false);
                s8 = __builtin_amdgcn_sdot4((int)q.y, 0x01010101, s8, false);
                s8 = __builtin_amdgcn_sdot4((int)q.z, 0x01010101, s8, false);
                s8 = __builtin_amdgcn_sdot4((int)q.w, 0x01010101, s8, false);
                s8 += dpp_i32<0xB1, 0xf>(s8);  // the other half of the chunk
                uint2 hi, lo;
                nibble_planes(q.x ^ 0x80808080u, q.y ^ 0x80808080u, hi.x, lo.x);
                nibble_planes(q.z ^ 0x80808080u, q.w ^ 0x80808080u, hi.y, lo.y);
                if (idx < xvecs) {
                    uint2 *slot = reinterpret_cast<uint2 *>(planes + (m * CP + (idx >> 1)) * 2);
                    slot[idx & 1] = hi;
                    slot[2 + (idx & 1)] = lo;
                    if ((idx & 1) == 0) xsum[m * CP + (idx >> 1)] = -8 * s8;
                }
            }
        }
    } else {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float amax = 0.f;
#pragma unroll
            for (int j = 0; j < XVN; ++j)
                if (j * THREADS < xvecs) amax = absmax8(v[m][j], amax);  // uniform: skip vectors past K
            amax = wave_max_to_lane63(amax);
            if (lane == 63) part[m * WAVES + wave] = amax;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float amax = part[m * WAVES];
#pragma unroll
            for (int wv = 1; wv < WAVES; ++wv) amax = fmaxf(amax, part[m * WAVES + wv]);
            const RowScale rs = row_scale(amax);
            if (threadIdx.x == 0) {
                xs_lds[m] = rs.sc;
                if (a.xs_out && block == 0 && m < a.M) a.xs_out[m] = rs.sc;
            }
#pragma unroll
            for (int j = 0; j < XVN; ++j) {
                if (j * THREADS >= xvecs) break;  // uniform
                const int idx = threadIdx.x + j * THREADS;  // 8 elements: a quarter of a chunk
                const uint2 q = quant8(v[m][j], rs);
                int s8 = __builtin_amdgcn_sdot4((int)q.x, 0x01010101, 0, false);
                s8 = __builtin_amdgcn_sdot4((int)q.y, 0x01010101, s8, false);
                s8 += dpp_i32<0xB1, 0xf>(s8);  // quad_perm [1,0,3,2]
                s8 += dpp_i32<0x4E, 0xf>(s8);  // quad_perm [2,3,0,1]
                uint32_t hi, lo;
                nibble_planes(q.x ^ 0x80808080u, q.y ^ 0x80808080u, hi, lo);
                if (idx < xvecs) {
                    uint32_t *slot = reinterpret_cast<uint32_t *>(planes + (m * CP + (idx >> 2)) * 2);
                    slot[idx & 3] = hi;
                    slot[4 + (idx & 3)] = lo;
                    if ((idx & 3) == 0) xsum[m * CP + (idx >> 2)] = -8 * s8;
                    if (a.xq_out && block == 0 && m < a.M)
                        reinterpret_cast<uint2 *>(a.xq_out + (size_t)m * a.K)[idx] = q;
                }
            }
        }
    }
    __syncthreads();

    // 5. integer group sums and the fp32 chain, load by load
    float total[M];
    float fr[M][S > 1 ? NL : 1];  // converted sums waiting for the chain to arrive (S > 1)
#pragma unroll
    for (int m = 0; m < M; ++m) total[m] = 0.f;
    auto extend = [&](int m, int j, float f) {
        total[m] = fmaf(f, wsr[j][0], total[m]);
        if constexpr (Q >= 2) total[m] = fmaf(dpp_f32<0x104, 0xf>(f), wsr[j][1], total[m]);  // row_shl:4
        if constexpr (Q >= 3) total[m] = fmaf(dpp_f32<0x108, 0xf>(f), wsr[j][2], total[m]);  // row_shl:8
        if constexpr (Q >= 4) total[m] = fmaf(dpp_f32<0x10C, 0xf>(f), wsr[j][3], total[m]);  // row_shl:12
    };
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        if constexpr (S > 1) {
#pragma unroll
            for (int m = 0; m < M; ++m) fr[m][j] = 0.f;  // loads past K: scale 0 as well
        }
        if constexpr (!EXACT)
            if ((j0 + j) * LPR >= nchunks) continue;  // uniform
        const uint32_t ww[4] = {w[j].x, w[j].y, w[j].z, w[j].w};
        uint32_t c8 = 0;  // 8 * (sum of the chunk's codes)
#pragma unroll
        for (int i = 0; i < 4; ++i) c8 = __builtin_amdgcn_udot8(ww[i], 0x88888888u, c8, false);
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const int slot = m * CP + (j0 + j) * LPR + c;
            const uint4 ph = planes[slot * 2], pl = planes[slot * 2 + 1];
            const uint32_t xh[4] = {ph.x, ph.y, ph.z, ph.w}, xl[4] = {pl.x, pl.y, pl.z, pl.w};
            uint32_t hi = 0, lo = (uint32_t)xsum[slot];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                hi = __builtin_amdgcn_udot8(ww[i], xh[i], hi, false);
                lo = __builtin_amdgcn_udot8(ww[i], xl[i], lo, false);
            }
            int s = (int)(((hi - c8) << 4) + lo);
            s += dpp_i32<0xB1, 0xf>(s);
            s += dpp_i32<0x4E, 0xf>(s);
            if constexpr (!EXACT) {
                if (a.group_acc) {  // uniform
                    const int g = (j0 + j) * Q + (c >> 2);
                    if ((c & 3) == 0 && g < a.G && n_raw < a.N && m < a.M)
                        a.group_acc[((size_t)m * a.G + g) * a.N + n] = s;
                }
            }
            if constexpr (S == 1)
                extend(m, j, (float)s);
            else
                fr[m][j] = (float)s;
        }
    }
    if constexpr (S > 1) {
        // the chain passes through the team's wavefronts in k order
#pragma unroll
        for (int t = 0; t < S; ++t) {
            if (part_s == t) {  // uniform
                if (t > 0) {
#pragma unroll
                    for (int m = 0; m < M; ++m) total[m] = carry[(team * M + m) * 16 + r];
                }
#pragma unroll
                for (int j = 0; j < NL; ++j)
#pragma unroll
                    for (int m = 0; m < M; ++m) extend(m, j, fr[m][j]);
                if (t < S - 1 && c == 0) {
#pragma unroll
                    for (int m = 0; m < M; ++m) carry[(team * M + m) * 16 + r] = total[m];
                }
            }
            if (t < S - 1) __syncthreads();
        }
        if (part_s != S - 1) return;
    }
    if (c == 0 && n_raw < a.N) {
#pragma unroll
        for (int m = 0; m < M; ++m)
            if (m < a.M) a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(total[m] * xs_lds[m]);
    }
}

template <int M, int LPR, int NL, bool PREQ, int S, int WAVES>
int launch(const Args &a, hipStream_t st) {
    constexpr int RPB = (WAVES / S) * (64 / LPR);
    constexpr int LDS_BYTES = Lds<M, S * NL * LPR, WAVES>::total;
    const dim3 grid((a.N + RPB - 1) / RPB), block(64 * WAVES);
    if (a.K == S * NL * LPR * 32 && !a.group_acc)
        gemv_w4a8_chain_kernel<M, LPR, NL, PREQ, true, S, WAVES><<<grid, block, LDS_BYTES, st>>>(a);
    else
        gemv_w4a8_chain_kernel<M, LPR, NL, PREQ, false, S, WAVES><<<grid, block, LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemv_w4a8");
}

// Loads per wavefront: the instantiations cover up to 20 (80 registers of weights).
template <int M, int LPR, bool PREQ, int S, int WAVES>
int dispatch_nl(const Args &a, hipStream_t st) {
    const int loads = ((a.K + LPR * 32 - 1) / (LPR * 32) + S - 1) / S;
    if (loads <= 2) return launch<M, LPR, 2, PREQ, S, WAVES>(a, st);
    if (loads <= 4) return launch<M, LPR, 4, PREQ, S, WAVES>(a, st);
    if (loads <= 5) return launch<M, LPR, 5, PREQ, S, WAVES>(a, st);
    if (loads <= 8) return launch<M, LPR, 8, PREQ, S, WAVES>(a, st);
    if (loads <= 10) return launch<M, LPR, 10, PREQ, S, WAVES>(a, st);
    if constexpr (LPR == 8 && S == 1) {
        if (loads <= 16) return launch<M, LPR, 16, PREQ, S, WAVES>(a, st);
        if (loads <= 20) return launch<M, LPR, 20, PREQ, S, WAVES>(a, st);
    }

    return CMI_E_UNSUPPORTED;
}

template <int M, bool PREQ>
int dispatch(const Args &a, int lanes, int split, int waves, hipStream_t st) {
    if (lanes == 8 && split == 1 && waves == 4) return dispatch_nl<M, 8, PREQ, 1, 4>(a, st);
    if (lanes == 8 && split == 1 && waves == 8) return dispatch_nl<M, 8, PREQ, 1, 8>(a, st);
    if (lanes == 16) {
        if (split == 1 && waves == 4) return dispatch_nl<M, 16, PREQ, 1, 4>(a, st);
        if (split == 1 && waves == 8) return dispatch_nl<M, 16, PREQ, 1, 8>(a, st);
        if (split == 1 && waves == 16) return dispatch_nl<M, 16, PREQ, 1, 16>(a, st);
        if (split == 2 && waves == 4) return dispatch_nl<M, 16, PREQ, 2, 4>(a, st);
        if (split == 4 && waves == 4) return dispatch_nl<M, 16, PREQ, 4, 4>(a, st);
        if (split == 2 && waves == 8) return dispatch_nl<M, 16, PREQ, 2, 8>(a, st);
        if (split == 4 && waves == 8) return dispatch_nl<M, 16, PREQ, 4, 8>(a, st);
        if (split == 4 && waves == 16) return dispatch_nl<M, 16, PREQ, 4, 16>(a, st);
        if (split == 8 && waves == 8) return dispatch_nl<M, 16, PREQ, 8, 8>(a, st);
        if (split == 8 && waves == 16) return dispatch_nl<M, 16, PREQ, 8, 16>(a, st);
    }
    return CMI_E_UNSUPPORTED;
}

}  // namespace

namespace cmi {

// Exactly one of x (bf16) and xq/xs (already quantised) is given.  `variant` = lanes per weight row
// (8, 16) + 100 * wavefronts sharing a row (1, 2, 4) + 10000 * wavefronts per workgroup (4, 8, 16).
// CMI_E_UNSUPPORTED (no error text) when the shape is outside the variant's range.
int gemv_w4a8_chain(const uint8_t *w4, const float *ws, const void *x, const int8_t *xq, const float *xs,
                    void *y, int32_t *group_acc, int8_t *xq_out, float *xs_out, int M, int N, int K,
                    int variant, void *stream) {
    const int lanes = variant % 100, split = variant / 100 % 100, waves = variant / 10000;
    if (M < 1 || M > 2 || K < GS || K % GS != 0 || N < 1) return CMI_E_UNSUPPORTED;
    Args a;
    a.w4 = w4;
    a.ws = ws;
    a.x = static_cast<const uint16_t *>(x);
    a.xq = xq;
    a.xs = xs;
    a.y = static_cast<uint16_t *>(y);
    a.group_acc = group_acc;
    a.xq_out = xq_out;
    a.xs_out = xs_out;
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = K / GS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x) return M <= 1 ? dispatch<1, false>(a, lanes, split, waves, st) : dispatch<2, false>(a, lanes, split, waves, st);
    return M <= 1 ? dispatch<1, true>(a, lanes, split, waves, st) : dispatch<2, true>(a, lanes, split, waves, st);
}

}  // namespace cmi
