// int8 weight-only GEMV for 1..16 activation rows: y = bf16(ws[n] * sum_k wq[n,k] x[m,k]).
//
// HBM-bound: the only large stream is the int8 weight, read exactly once with
// 16-byte loads that are contiguous across the wavefront (1 KiB per
// wave-load).  No MFMA: int8 is widened in registers (SDWA convert + byte
// permute to packed bf16, exact for |w| <= 127) and multiplied against packed
// bf16 activations with v_dot2c_f32_bf16, fp32 accumulation.
//
// Canonical summation order (what makes a batched row bit-identical to the
// single-row call, whatever blocking the launcher picks):
//   - K is cut into segments of 1024 (64 lanes x 16 elements); lane l of
//     segment s owns elements [s*1024 + l*16, +16);
//   - a lane's 16 products are accumulated pairwise in k order from 0.f
//     (eight chained dot2);
//   - the 64 lane partials are summed by the fixed DPP tree wave_sum_to_lane63;
//   - the segment totals are added in ascending segment order, starting from
//     segment 0's total (not from 0.f);
//   - the per-row weight scale multiplies that sum once, then one bf16 rounding.
//
// Blocking: a team of KW wavefronts shares R weight rows and walks K in trips
// of KW*CH segments; in a trip, wavefront kw owns CH consecutive segments.  The
// activations of those segments sit in registers (M*CH*8 VGPRs); the weights of
// all R rows are issued before any is consumed (R*CH loads of 1 KiB in flight
// per wavefront).  The final lane of each team adds the segment totals.
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
    int nchunks;  // K / 16
    int nseg;     // ceil(nchunks / 64)
    int KW;       // wavefronts per team
    int teams;    // teams per workgroup
    int iters;    // K-loop trips; a team covers KW*CH segments per trip
};

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

template <int M, int R, int CH>
__global__ void __launch_bounds__(256)
gemv_w8a16_kernel(const GemvArgs a) {
    extern __shared__ float red[];  // [teams][iters*KW*CH][R*M]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int team = wave / a.KW;
    const int kw = wave - team * a.KW;
    const int n0 = (blockIdx.x * a.teams + team) * R;
    float *team_red = red + (size_t)team * (a.iters * a.KW * CH) * (R * M);

    const u32x4 *wrow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int n = n0 + r < a.N ? n0 + r : a.N - 1;
        wrow[r] = reinterpret_cast<const u32x4 *>(a.wq + (size_t)n * a.K);
    }

    for (int it = 0; it < a.iters; ++it) {
        // Chunk (16 elements) owned by this lane in each of this trip's segments.
        const int seg0 = (it * a.KW + kw) * CH;
        int chunk[CH];
        bool live[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            chunk[j] = (seg0 + j) * 64 + lane;
            live[j] = chunk[j] < a.nchunks;
        }

        // Weights first: every load of the row block is issued before any is consumed.
        u32x4 wr[R][CH];
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int j = 0; j < CH; ++j)
                wr[r][j] = live[j] ? __builtin_nontemporal_load(wrow[r] + chunk[j])
                                   : u32x4{0, 0, 0, 0};
        }

        // Activations: M rows x CH chunks x 16 bf16, packed pairs (cache resident).
        uint4 xr[M][CH][2];
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const int mrow = m < a.M ? m : a.M - 1;
            const uint4 *xp = reinterpret_cast<const uint4 *>(a.x + (size_t)mrow * a.K);
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                if (live[j]) {
                    xr[m][j][0] = xp[2 * chunk[j]];
                    xr[m][j][1] = xp[2 * chunk[j] + 1];
                } else {
                    xr[m][j][0] = make_uint4(0, 0, 0, 0);
                    xr[m][j][1] = make_uint4(0, 0, 0, 0);
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                bf16x2_t wb[8];
                widen4(wr[r][j].x, wb[0], wb[1]);
                widen4(wr[r][j].y, wb[2], wb[3]);
                widen4(wr[r][j].z, wb[4], wb[5]);
                widen4(wr[r][j].w, wb[6], wb[7]);
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const uint32_t xv[8] = {xr[m][j][0].x, xr[m][j][0].y, xr[m][j][0].z,
                                            xr[m][j][0].w, xr[m][j][1].x, xr[m][j][1].y,
                                            xr[m][j][1].z, xr[m][j][1].w};
                    float acc = 0.f;
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        acc = __builtin_amdgcn_fdot2_f32_bf16(
                            wb[i], __builtin_bit_cast(bf16x2_t, xv[i]), acc, false);
                    acc = wave_sum_to_lane63(acc);
                    if (lane == 63) team_red[(seg0 + j) * (R * M) + r * M + m] = acc;
                }
            }
        }
    }
    __syncthreads();

    if (kw == 0 && lane < R * M) {
        const int r = lane / M, m = lane - r * M;
        const int n = n0 + r;
        if (n < a.N && m < a.M) {
            float total = team_red[lane];
            for (int s = 1; s < a.nseg; ++s) total += team_red[s * (R * M) + lane];
            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(a.ws[n] * total);
        }
    }
}

struct Plan {
    int mt, r, ch, kw, teams, iters;
};

// Blocking is a pure function of (M, N, K); it never changes results.
Plan make_plan(int M, int N, int K) {
    Plan p;
    p.mt = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    const int chmax = p.mt <= 4 ? 4 : p.mt <= 8 ? 2 : 1;
    const int nseg = (K / 16 + 63) / 64;
    // Rows per team: enough wavefronts to cover the chip a few times over.
    int r = p.mt >= 16 ? 8 : 4;
    // Search (KW, CH, iters): up to a quarter of padding is accepted for fewer
    // trips (more loads in flight); then least padding, then fewest wavefronts.
    long best = -1;
    p.kw = 1; p.ch = 1; p.iters = nseg;
    for (int kw = 1; kw <= 4; kw *= 2) {
        for (int ch = 1; ch <= chmax; ++ch) {
            const int per_trip = kw * ch;
            const int iters = (nseg + per_trip - 1) / per_trip;
            const int waste = iters * per_trip - nseg;
            if (waste * 4 > nseg && waste > 1) continue;
            const long cost = (long)iters * 10000 + waste * 100 + kw;
            if (best < 0 || cost < best) {
                best = cost;
                p.kw = kw; p.ch = ch; p.iters = iters;
            }
        }
    }
    p.teams = 4 / p.kw;
    const long target_waves = 256L * 8;
    while (r > 1 && (long)((N + r - 1) / r) * p.kw < target_waves) r >>= 1;
    if (p.mt * r > 64) r = 64 / p.mt > 0 ? 64 / p.mt : 1;
    p.r = r;
    return p;
}

template <int M, int R, int CH>
int launch(const GemvArgs &a, hipStream_t st) {
    const int rows_per_block = R * a.teams;
    const dim3 grid((a.N + rows_per_block - 1) / rows_per_block);
    const dim3 block(64 * a.KW * a.teams);
    const size_t lds = sizeof(float) * a.teams * (a.iters * a.KW * CH) * R * M;
    gemv_w8a16_kernel<M, R, CH><<<grid, block, lds, st>>>(a);
    return check_launch("cmi_gemv_w8a16");
}

template <int M, int R>
int dispatch_ch(const GemvArgs &a, int ch, hipStream_t st) {
    constexpr int CHMAX = M <= 4 ? 4 : M <= 8 ? 2 : 1;
    if (ch == 1) return launch<M, R, 1>(a, st);
    if constexpr (CHMAX >= 2) if (ch == 2) return launch<M, R, 2>(a, st);
    if constexpr (CHMAX >= 4) {
        if (ch == 3) return launch<M, R, 3>(a, st);
        if (ch == 4) return launch<M, R, 4>(a, st);
    }
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: no kernel for M-tile %d with %d chunks", M, ch);
}

template <int M>
int dispatch_r(const GemvArgs &a, const Plan &p, hipStream_t st) {
    switch (p.r) {
        case 1: return dispatch_ch<M, 1>(a, p.ch, st);
        case 2: return dispatch_ch<M, 2>(a, p.ch, st);
        case 4: return dispatch_ch<M, 4>(a, p.ch, st);
        case 8: if constexpr (M * 8 <= 64) return dispatch_ch<M, 8>(a, p.ch, st);
    }
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: no kernel for %d rows per team", p.r);
}

}  // namespace

extern "C" int cmi_gemv_w8a16(const int8_t *wq, const float *ws, const void *x, void *y,
                              int M, int N, int K, void *stream) {
    CMI_REQUIRE(wq && ws && x && y, CMI_E_ARG, "cmi_gemv_w8a16: null pointer");
    CMI_REQUIRE(M >= 1 && M <= 16, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: M=%d outside 1..16", M);
    CMI_REQUIRE(N >= 1 && K >= 16, CMI_E_ARG, "cmi_gemv_w8a16: bad shape N=%d K=%d", N, K);
    CMI_REQUIRE(K % 16 == 0, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: K=%d is not a multiple of 16", K);
    CMI_REQUIRE(K <= (1 << 20), CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: K=%d above 2^20", K);
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
    a.KW = p.kw;
    a.teams = p.teams;
    a.iters = p.iters;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (p.mt) {
        case 1: return dispatch_r<1>(a, p, st);
        case 2: return dispatch_r<2>(a, p, st);
        case 4: return dispatch_r<4>(a, p, st);
        case 8: return dispatch_r<8>(a, p, st);
        default: return dispatch_r<16>(a, p, st);
    }
}
