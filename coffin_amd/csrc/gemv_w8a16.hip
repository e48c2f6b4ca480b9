// int8 weight-only GEMV for 1..16 activation rows: y = bf16(ws[n] * sum_k wq[n,k] x[m,k]).
//
// HBM-bound: the only large stream is the int8 weight, read exactly once with
// 16-byte loads that are contiguous across the wavefront (1 KiB per
// wave-load).  No MFMA: int8 is widened in registers (SDWA convert + byte
// permute to packed bf16, exact for |w| <= 127) and multiplied against packed
// bf16 activations with v_dot2c_f32_bf16, fp32 accumulation.
//
// Canonical summation order (what makes a batched row bit-identical to the
// single-row call, whatever blocking the launcher picks); it depends on K only:
//   - K is cut into segments of 1024 (64 lanes x 16 elements); lane l of
//     segment s owns elements [s*1024 + l*16, +16);
//   - U consecutive segments form a unit (U = unit_segments(K), 1..4);
//   - inside a unit a lane accumulates its products in k order into one fp32
//     chain that starts at 0.f (eight chained dot2 per segment, segments
//     ascending);
//   - the 64 lane chains of a unit are summed by the fixed DPP tree
//     wave_sum_to_lane63;
//   - unit totals are added in ascending unit order, starting from unit 0's
//     total (not from 0.f);
//   - the per-row weight scale multiplies that sum once, then one bf16 rounding.
//
// Execution: one wavefront = (block of R weight rows, one unit of K).  All of a
// wavefront's weight loads are issued up front and there are many small
// wavefronts (R = 2: 2 KiB x CHT in flight each, ~70 VGPRs), which is what keeps
// HBM saturated from the first microsecond to the last: the hardware dispatcher
// back-fills retiring wavefronts, so late memory service of one wavefront never
// idles the rest.  A unit wider than the register budget of M rows is walked in
// sub-trips with the next sub-trip's loads in flight.  When K spans several
// units the wavefronts of a workgroup each take one unit of the same rows and
// the unit totals meet in LDS (summed in unit order by one lane per output);
// otherwise there is no LDS and no barrier: lane 63, which holds the tree
// result, scales and stores.
#include "common.hpp"

namespace {

using namespace cmi;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct GemvArgs {
    const int8_t *wq;
    const float *ws;
    const uint16_t *x;
    uint16_t *y;
    int M, N, K;
    int nchunks;    // K / 16
    int nseg;       // ceil(nchunks / 64)
    int unit;       // segments per unit (canonical, from K)
    int units;      // ceil(nseg / unit)
    int subtrips;   // ceil(unit / CHT)
    int nblocks;    // ceil(N / R)
    int teams;      // row blocks per workgroup (units == 1: 4, else 1)
};

// Segments per unit: the largest of 4,3,2,1 that pads K by at most a fifth.
inline int unit_segments(int nseg) {
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

template <int M, int CHT>
struct XStage {
    uint4 x[M][CHT][2];
};

template <int R, int CHT>
struct WStage {
    u32x4 w[R][CHT];
};

// MODE 0: K is one unit that fits one sub-trip (no loop, no LDS, no barrier).
// MODE 1: several units, each one sub-trip (all loads up front, totals via LDS).
// MODE 2: general: units walked in pipelined sub-trips.
template <int M, int R, int CHT, int MODE>
__global__ void __launch_bounds__(256)
gemv_w8a16_kernel(const GemvArgs a) {
    constexpr bool SINGLE = MODE == 0;
    extern __shared__ float unit_total[];  // [units][R*M], only when units > 1
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int rb = SINGLE ? blockIdx.x * a.teams + wave : blockIdx.x;
    const bool idle = rb >= a.nblocks;  // only in the last workgroup of a SINGLE launch
    int u = SINGLE ? 0 : wave;          // unit in hand; wavefronts stride over the units
    int seg_end = min((u + 1) * a.unit, a.nseg);

    const u32x4 *wrow[R];
    float scale[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int n = rb * R + r;
        n = n < a.N ? n : a.N - 1;
        wrow[r] = reinterpret_cast<const u32x4 *>(a.wq + (size_t)n * a.K);
    }

    // Loads are unconditional: a dead chunk's address is clamped to the row's
    // last chunk and its activations are zeroed, so nothing branches between a
    // load and the arithmetic it overlaps.
    auto load_w = [&](WStage<R, CHT> &s, int t) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < CHT; ++j) {
                const int chunk = (u * a.unit + t * CHT + j) * 64 + lane;
                s.w[r][j] = __builtin_nontemporal_load(wrow[r] + min(chunk, a.nchunks - 1));
            }
    };
    auto load_x = [&](XStage<M, CHT> &s, int t) {
#pragma unroll
        for (int j = 0; j < CHT; ++j) {
            const int seg = u * a.unit + t * CHT + j;
            const int chunk = seg * 64 + lane;
            const bool live = seg < seg_end && chunk < a.nchunks;
            const int safe = min(chunk, a.nchunks - 1);
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const int mrow = m < a.M ? m : a.M - 1;
                const uint4 *xp = reinterpret_cast<const uint4 *>(a.x + (size_t)mrow * a.K);
                const uint4 lo = xp[2 * safe], hi = xp[2 * safe + 1];
                s.x[m][j][0] = live ? lo : make_uint4(0, 0, 0, 0);
                s.x[m][j][1] = live ? hi : make_uint4(0, 0, 0, 0);
            }
        }
    };

    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = 0.f;

    auto compute = [&](const WStage<R, CHT> &ws_, const XStage<M, CHT> &xs_) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int j = 0; j < CHT; ++j) {
                bf16x2_t wb[8];
                widen4(ws_.w[r][j].x, wb[0], wb[1]);
                widen4(ws_.w[r][j].y, wb[2], wb[3]);
                widen4(ws_.w[r][j].z, wb[4], wb[5]);
                widen4(ws_.w[r][j].w, wb[6], wb[7]);
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const uint32_t xv[8] = {xs_.x[m][j][0].x, xs_.x[m][j][0].y, xs_.x[m][j][0].z,
                                            xs_.x[m][j][0].w, xs_.x[m][j][1].x, xs_.x[m][j][1].y,
                                            xs_.x[m][j][1].z, xs_.x[m][j][1].w};
                    float v = acc[r][m];
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        v = __builtin_amdgcn_fdot2_f32_bf16(wb[i], __builtin_bit_cast(bf16x2_t, xv[i]),
                                                            v, false);
                    acc[r][m] = v;
                }
            }
        }
    };

    for (; SINGLE || u < a.units; u += nwaves) {
        if (idle) break;
        seg_end = min((u + 1) * a.unit, a.nseg);
        WStage<R, CHT> w0;
        XStage<M, CHT> x0;
        load_w(w0, 0);
        load_x(x0, 0);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int n = rb * R + r;
            scale[r] = a.ws[n < a.N ? n : a.N - 1];
        }
        if constexpr (MODE != 2) {
            compute(w0, x0);
        } else {
            WStage<R, CHT> w1;
            XStage<M, CHT> x1;
            // sub-trips of the unit, next one in flight while this one is consumed
            int t = 0;
            for (; t + 2 < a.subtrips; t += 2) {
                load_w(w1, t + 1);
                load_x(x1, t + 1);
                compute(w0, x0);
                load_w(w0, t + 2);
                load_x(x0, t + 2);
                compute(w1, x1);
            }
            if (t + 1 < a.subtrips) {
                load_w(w1, t + 1);
                load_x(x1, t + 1);
                compute(w0, x0);
                compute(w1, x1);
            } else {
                compute(w0, x0);
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) acc[r][m] = wave_sum_to_lane63(acc[r][m]);
        if constexpr (SINGLE) break;
        if (a.units > 1) {
            // unit totals meet in LDS; one lane per output adds them in unit order below
            if (lane == 63) {
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int m = 0; m < M; ++m) unit_total[u * (R * M) + r * M + m] = acc[r][m];
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int m = 0; m < M; ++m) acc[r][m] = 0.f;
        } else {
            break;
        }
    }

    if (SINGLE || a.units == 1) {
        if (!idle && lane == 63) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int n = rb * R + r;
                if (n < a.N) {
#pragma unroll
                    for (int m = 0; m < M; ++m)
                        if (m < a.M)
                            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(scale[r] * acc[r][m]);
                }
            }
        }
        return;
    }

    __syncthreads();
    if (wave == 0 && lane < R * M) {
        const int r = lane / M, m = lane - r * M;
        const int n = rb * R + r;
        if (n < a.N && m < a.M) {
            float total = unit_total[lane];
            for (int v = 1; v < a.units; ++v) total += unit_total[v * (R * M) + lane];
            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(a.ws[n] * total);
        }
    }
}

struct Plan {
    int mt, r, cht;
    bool single;
};

//: Most K-units one launch handles (LDS holds one total per unit and output).
constexpr int MAX_UNITS = 256;

// Blocking is a pure function of (M, N, K); it never changes results.
Plan make_plan(int M, int N, int K) {
    Plan p;
    p.mt = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    const int nseg = (K / 16 + 63) / 64;
    const int unit = unit_segments(nseg);
    const int units = (nseg + unit - 1) / unit;
    const int chmax = p.mt <= 2 ? 4 : p.mt <= 4 ? 3 : 1;
    p.cht = unit < chmax ? unit : chmax;
    // balance the sub-trips of a unit (e.g. 4 segments at CHT<=3 -> 2 + 2)
    const int subtrips = (unit + p.cht - 1) / p.cht;
    p.cht = (unit + subtrips - 1) / subtrips;
    p.single = nseg <= p.cht;
    // Two rows per wavefront; one when that would leave fewer than ~8 wavefronts per CU.
    p.r = p.mt >= 16 ? 1 : 2;
    if ((long)((N + 1) / 2) * units < 2048) p.r = 1;
    return p;
}

template <int M, int R, int CHT, int MODE>
int launch(GemvArgs &a, hipStream_t st) {
    constexpr bool SINGLE = MODE == 0;
    a.nblocks = (a.N + R - 1) / R;
    a.subtrips = (a.unit + CHT - 1) / CHT;
    a.teams = SINGLE ? 4 : 1;
    const dim3 grid(SINGLE ? (a.nblocks + 3) / 4 : a.nblocks);
    const dim3 block(SINGLE ? 256 : 64 * (a.units < 4 ? a.units : 4));
    const size_t lds = (SINGLE || a.units == 1) ? 0 : sizeof(float) * a.units * R * M;
    gemv_w8a16_kernel<M, R, CHT, MODE><<<grid, block, lds, st>>>(a);
    return check_launch("cmi_gemv_w8a16");
}

template <int M, int R, int CHT>
int dispatch_x(GemvArgs &a, const Plan &p, hipStream_t st) {
    if (p.single) return launch<M, R, CHT, 0>(a, st);
    if ((a.unit + CHT - 1) / CHT == 1) return launch<M, R, CHT, 1>(a, st);
    return launch<M, R, CHT, 2>(a, st);
}

template <int M, int R>
int dispatch_ch(GemvArgs &a, const Plan &p, hipStream_t st) {
    constexpr int CHMAX = M <= 2 ? 4 : M <= 4 ? 3 : 1;
    if (p.cht == 1) return dispatch_x<M, R, 1>(a, p, st);
    if constexpr (CHMAX >= 2) if (p.cht == 2) return dispatch_x<M, R, 2>(a, p, st);
    if constexpr (CHMAX >= 3) if (p.cht == 3) return dispatch_x<M, R, 3>(a, p, st);
    if constexpr (CHMAX >= 4) if (p.cht == 4) return dispatch_x<M, R, 4>(a, p, st);
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: no kernel for M-tile %d with %d chunks", M, p.cht);
}

template <int M>
int dispatch_r(GemvArgs &a, const Plan &p, hipStream_t st) {
    switch (p.r) {
        case 1: return dispatch_ch<M, 1>(a, p, st);
        case 2: return dispatch_ch<M, 2>(a, p, st);
    }
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: no kernel for %d rows per block", p.r);
}

}  // namespace

extern "C" int cmi_gemv_w8a16(const int8_t *wq, const float *ws, const void *x, void *y,
                              int M, int N, int K, void *stream) {
    CMI_REQUIRE(wq && ws && x && y, CMI_E_ARG, "cmi_gemv_w8a16: null pointer");
    CMI_REQUIRE(M >= 1 && M <= 16, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: M=%d outside 1..16", M);
    CMI_REQUIRE(N >= 1 && K >= 16, CMI_E_ARG, "cmi_gemv_w8a16: bad shape N=%d K=%d", N, K);
    CMI_REQUIRE(K % 16 == 0, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: K=%d is not a multiple of 16", K);
    CMI_REQUIRE(aligned(wq, 16) && aligned(x, 16) && aligned(y, 2) && aligned(ws, 4), CMI_E_ARG,
                "cmi_gemv_w8a16: wq and x must be 16-byte aligned");
    const Plan p = make_plan(M, N, K);
    GemvArgs a;
    a.wq = wq;
    a.ws = ws;
    a.x = static_cast<const uint16_t *>(x);
    a.y = static_cast<uint16_t *>(y);
    a.M = M;
    a.N = N;
    a.K = K;
    a.nchunks = K / 16;
    a.nseg = (a.nchunks + 63) / 64;
    a.unit = unit_segments(a.nseg);
    a.units = (a.nseg + a.unit - 1) / a.unit;
    CMI_REQUIRE(a.units <= MAX_UNITS, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: K=%d above %d", K,
                MAX_UNITS * 4096);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (p.mt) {
        case 1: return dispatch_r<1>(a, p, st);
        case 2: return dispatch_r<2>(a, p, st);
        case 4: return dispatch_r<4>(a, p, st);
        case 8: return dispatch_r<8>(a, p, st);
        default: return dispatch_r<16>(a, p, st);
    }
}
