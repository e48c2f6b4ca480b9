// W4A8 GEMV for 1..16 activation rows on the re-laid-out int4 weight.
//
//   sum_g  = sum_{k in group g} xq[m,k] * (code(n,k) - 8)     int32, exact
//   total  = fma((float)sum_g, ws[n,g], total)                 g = 0,1,.. from 0.f
//   y[m,n] = bf16(total * xs[m])
//
// HBM-bound on the packed weight (half a byte per element), read once with
// 16-byte loads; a half-wavefront (32 lanes, 512 contiguous bytes) walks one
// output row so that 2560-wide rows (1280 B) fill whole loads.  No MFMA:
// nibbles are split with two AND/shift ops per word into the byte operands of
// v_dot4_i32_i8, whose accumulator starts at -8 * sum(xq) so the unsigned
// codes never need re-biasing.  Four adjacent lanes own one group of 128 k;
// their int32 partials are added with two DPP quad permutes.  The fp32 part of
// the arithmetic is a strict chain over the groups and is order sensitive, so
// group sums go through LDS and one lane per (row, m) walks them in order:
// the result does not depend on how K was split over wavefronts or trips.
#include "quant_math.hpp"

namespace {

using namespace cmi;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GS = 128;  // group size the fast kernels are built for; the general kernel below also takes 64 and 256
constexpr int FUSED_MAX_ROWS = 4;  // activation rows the fused-quantiser variant takes

struct W4Args {
    const uint8_t *w4;
    const float *ws;
    const int8_t *xq;
    const float *xs;
    const uint16_t *xb;   // bf16 activations (fused quantiser) or null
    int8_t *xq_out;       // optional copies of the fused quantiser's results
    float *xs_out;
    uint16_t *y;
    int32_t *group_acc;
    int M, N, K;
    int G;        // K / group size
    int nchunks;  // K / 32: 16-byte chunks per row
    int KW, teams, iters;
};

// XV == 0: activations arrive quantised (a.xq, a.xs).  XV > 0: they arrive as bf16
// (a.xb) and every workgroup (256 threads) quantises them into LDS first -- XV
// 16-byte vectors per thread and row -- with the arithmetic of the stand-alone
// quantiser; the bf16 loads are issued before anything else and the weight
// stream hides the work.  Saves a launch and the int8 round trip through memory.
// LG: log2(group size / 32) -- 1, 2, 3 for groups of 64, 128, 256: a lane's 16-byte load is 32 k,
// so 2, 4 or 8 adjacent lanes own a group and their partial sums meet in one, two or three DPP steps.
template <int M, int R2, int CH, int XV, int LG = 2>
__global__ void __launch_bounds__(256)
gemv_w4a8_kernel(const W4Args a) {
    constexpr int ROWS = 2 * R2;
    constexpr int GPH = 32 >> LG;  // groups per half-wavefront load (32 chunks of 32 k)
    static_assert(LG >= 1 && LG <= 3 && (LG == 2 || XV == 0), "group sizes 64, 128, 256; the fused quantiser only with 128");
    extern __shared__ int32_t sums_base[];  // [fused: M*K int8, M scales, M*4 partial maxima] [teams][groups][ROWS*M]
    int8_t *xq_lds = reinterpret_cast<int8_t *>(sums_base);
    float *xs_lds = reinterpret_cast<float *>(xq_lds + (XV ? (size_t)M * a.K : 0));
    int32_t *sums = reinterpret_cast<int32_t *>(xs_lds + (XV ? M * 5 : 0));
    if constexpr (XV > 0) {
        const int xvecs = a.K / 8;
        uint4 v[M][XV];
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const uint4 *xg = reinterpret_cast<const uint4 *>(a.xb + (size_t)(m < a.M ? m : a.M - 1) * a.K);
#pragma unroll
            for (int j = 0; j < XV; ++j) {
                const int idx = threadIdx.x + j * 256;
                v[m][j] = idx < xvecs ? xg[idx] : make_uint4(0, 0, 0, 0);
            }
        }
        float *part = xs_lds + M;
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float amax = 0.f;
#pragma unroll
            for (int j = 0; j < XV; ++j) amax = absmax8(v[m][j], amax);
            amax = wave_max_to_lane63(amax);
            if ((threadIdx.x & 63) == 63) part[m * 4 + (threadIdx.x >> 6)] = amax;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float amax = fmaxf(fmaxf(part[m * 4], part[m * 4 + 1]), fmaxf(part[m * 4 + 2], part[m * 4 + 3]));
            const RowScale rs = row_scale(amax);
            const float sc = rs.sc;
            if (threadIdx.x == 0) {
                xs_lds[m] = sc;
                if (a.xs_out && blockIdx.x == 0 && m < a.M) a.xs_out[m] = sc;
            }
#pragma unroll
            for (int j = 0; j < XV; ++j) {
                const int idx = threadIdx.x + j * 256;
                if (idx < xvecs) {
                    const uint2 q = quant8(v[m][j], rs);
                    reinterpret_cast<uint2 *>(xq_lds + (size_t)m * a.K)[idx] = q;
                    if (a.xq_out && blockIdx.x == 0 && m < a.M)
                        reinterpret_cast<uint2 *>(a.xq_out + (size_t)m * a.K)[idx] = q;
                }
            }
        }
        __syncthreads();
    }
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5, hl = lane & 31;
    const int wave = threadIdx.x >> 6;
    const int team = wave / a.KW;
    const int kw = wave - team * a.KW;
    const int n0 = (blockIdx.x * a.teams + team) * ROWS;
    int32_t *team_sums = sums + (size_t)team * (a.iters * a.KW * CH * GPH) * (ROWS * M);
    const int row_bytes = a.K / 2;

    const u32x4 *wrow[R2];
#pragma unroll
    for (int rr = 0; rr < R2; ++rr) {
        int n = n0 + 2 * rr + half;
        n = n < a.N ? n : a.N - 1;
        wrow[rr] = reinterpret_cast<const u32x4 *>(a.w4 + (size_t)n * row_bytes);
    }

    for (int it = 0; it < a.iters; ++it) {
        const int hs0 = (it * a.KW + kw) * CH;
        int chunk[CH];
        bool live[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            chunk[j] = (hs0 + j) * 32 + hl;
            live[j] = chunk[j] < a.nchunks;
        }

        u32x4 wr[R2][CH];
#pragma unroll
        for (int rr = 0; rr < R2; ++rr)
#pragma unroll
            for (int j = 0; j < CH; ++j)
                wr[rr][j] = live[j] ? __builtin_nontemporal_load(wrow[rr] + chunk[j]) : u32x4{0, 0, 0, 0};

        // Activations of this lane's chunks: 32 int8 per (m, chunk), and the
        // accumulator start value -8 * sum of those 32.
        uint4 xr[M][CH][2];
        int xinit[M][CH];
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const int mrow = m < a.M ? m : a.M - 1;
            const uint4 *xp = XV ? reinterpret_cast<const uint4 *>(xq_lds + (size_t)m * a.K)
                                 : reinterpret_cast<const uint4 *>(a.xq + (size_t)mrow * a.K);
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                if (live[j]) {
                    xr[m][j][0] = xp[2 * chunk[j]];
                    xr[m][j][1] = xp[2 * chunk[j] + 1];
                } else {
                    xr[m][j][0] = make_uint4(0, 0, 0, 0);
                    xr[m][j][1] = make_uint4(0, 0, 0, 0);
                }
                const uint32_t xv[8] = {xr[m][j][0].x, xr[m][j][0].y, xr[m][j][0].z, xr[m][j][0].w,
                                        xr[m][j][1].x, xr[m][j][1].y, xr[m][j][1].z, xr[m][j][1].w};
                int s = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) s = __builtin_amdgcn_sdot4((int)xv[i], 0x01010101, s, false);
                xinit[m][j] = -8 * s;
            }
        }

#pragma unroll
        for (int rr = 0; rr < R2; ++rr) {
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                const uint32_t w[4] = {wr[rr][j].x, wr[rr][j].y, wr[rr][j].z, wr[rr][j].w};
                uint32_t op[8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    op[2 * i] = w[i] & 0x0F0F0F0Fu;
                    op[2 * i + 1] = (w[i] >> 4) & 0x0F0F0F0Fu;
                }
                const int group = chunk[j] >> LG;
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const uint32_t xv[8] = {xr[m][j][0].x, xr[m][j][0].y, xr[m][j][0].z,
                                            xr[m][j][0].w, xr[m][j][1].x, xr[m][j][1].y,
                                            xr[m][j][1].z, xr[m][j][1].w};
                    int acc = xinit[m][j];
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        acc = __builtin_amdgcn_sdot4((int)op[i], (int)xv[i], acc, false);
                    acc += dpp_i32<0xB1, 0xf>(acc);                           // quad_perm [1,0,3,2]
                    if constexpr (LG >= 2) acc += dpp_i32<0x4E, 0xf>(acc);    // quad_perm [2,3,0,1]
                    if constexpr (LG >= 3) acc += dpp_i32<0x141, 0xf>(acc);   // row_half_mirror: the other quad of 8 lanes
                    if ((hl & ((1 << LG) - 1)) == 0 && live[j])
                        team_sums[group * (ROWS * M) + (2 * rr + half) * M + m] = acc;
                }
            }
        }
    }
    __syncthreads();

    if (kw == 0 && lane < ROWS * M) {
        const int r = lane / M, m = lane - r * M;
        const int n = n0 + r;
        if (n < a.N && m < a.M) {
            const float *wsn = a.ws + (size_t)n * a.G;
            float total = 0.f;
            for (int g = 0; g < a.G; ++g) {
                const int s = team_sums[g * (ROWS * M) + lane];
                if (a.group_acc) a.group_acc[((size_t)m * a.G + g) * a.N + n] = s;
                total = fmaf((float)s, wsn[g], total);
            }
            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(total * (XV ? xs_lds[m] : a.xs[m]));
        }
    }
}

struct Plan {
    int mt, r2, ch, kw, teams, iters;
};

// lg: log2(group size / 32).  Group sizes other than 128 are served by fewer instantiations (one
// row pair per wavefront, at most two chunks per trip).
Plan make_plan(int M, int N, int K, int lg) {
    Plan p;
    p.mt = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    const int gph = 32 >> lg;
    int chmax = p.mt <= 4 ? 4 : p.mt <= 8 ? 2 : 1;
    if (lg != 2 && chmax > 2) chmax = 2;
    const int nhseg = (K / 32 + 31) / 32;
    // Up to a quarter of padding is accepted for fewer trips (more loads in
    // flight); then least padding, then fewest wavefronts per team.
    long best = -1;
    p.kw = 1; p.ch = 1; p.iters = nhseg;
    for (int kw = 1; kw <= 4; kw *= 2) {
        for (int ch = 1; ch <= chmax; ++ch) {
            const int per_trip = kw * ch;
            const int iters = (nhseg + per_trip - 1) / per_trip;
            const int waste = iters * per_trip - nhseg;
            if (waste * 4 > nhseg && waste > 1) continue;
            const long cost = (long)iters * 10000 + waste * 100 + kw;
            if (best < 0 || cost < best) {
                best = cost;
                p.kw = kw; p.ch = ch; p.iters = iters;
            }
        }
    }
    p.teams = 4 / p.kw;
    int r2 = 2;
    const long target_waves = 256L * 8;
    while (r2 > 1 && (long)((N + 2 * r2 - 1) / (2 * r2)) * p.kw < target_waves) r2 >>= 1;
    while (2 * r2 * p.mt > 64) r2 >>= 1;
    p.r2 = r2 < 1 || lg != 2 ? 1 : r2;
    // Group sums of a whole team live in LDS; shrink the team count, then the
    // row block, until they fit comfortably.
    auto lds_bytes = [&]() {
        return (size_t)4 * p.teams * (p.iters * p.kw * p.ch * gph) * (2 * p.r2 * p.mt);
    };
    while (lds_bytes() > 48 * 1024 && p.teams > 1) p.teams >>= 1;
    while (lds_bytes() > 48 * 1024 && p.r2 > 1) p.r2 >>= 1;
    return p;
}

template <int M, int R2, int CH, int XV, int LG = 2>
int launch_xv(const W4Args &a, hipStream_t st) {
    const int rows_per_block = 2 * R2 * a.teams;
    const dim3 grid((a.N + rows_per_block - 1) / rows_per_block);
    const size_t lds = sizeof(int32_t) * a.teams * (a.iters * a.KW * CH * (32 >> LG)) * (2 * R2 * M) +
                       (XV ? (size_t)M * a.K + sizeof(float) * M * 5 : 0);
    if (lds > 64 * 1024)
        return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w4a8: K=%d needs %zu bytes of LDS", a.K, lds);
    gemv_w4a8_kernel<M, R2, CH, XV, LG><<<grid, dim3(64 * a.KW * a.teams), lds, st>>>(a);
    return check_launch("cmi_gemv_w4a8");
}

// Groups of 64 or 256: quantised activations only, one row pair per wavefront, one or two chunks per trip.
template <int M>
int launch_other_group(const W4Args &a, int ch, int lg, hipStream_t st) {
    if constexpr (M <= 8) {
        if (ch == 2) return lg == 1 ? launch_xv<M, 1, 2, 0, 1>(a, st) : launch_xv<M, 1, 2, 0, 3>(a, st);
    }
    return lg == 1 ? launch_xv<M, 1, 1, 0, 1>(a, st) : launch_xv<M, 1, 1, 0, 3>(a, st);
}

template <int M, int R2, int CH>
int launch(const W4Args &a, hipStream_t st) {
    if (!a.xb) return launch_xv<M, R2, CH, 0>(a, st);
    if constexpr (M <= FUSED_MAX_ROWS) {
        // the fused prologue is written for 256 threads
        if (a.KW * a.teams != 4)
            return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w4a8_bf16: K=%d leaves a workgroup of %d wavefronts", a.K,
                        a.KW * a.teams);
        const int xv = (a.K / 8 + 255) / 256;
        if (xv <= 2) return launch_xv<M, R2, CH, 2>(a, st);
        if (xv <= 5) return launch_xv<M, R2, CH, 5>(a, st);
        if (xv <= 8) return launch_xv<M, R2, CH, 8>(a, st);
    }
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w4a8_bf16: M=%d K=%d outside the fused kernel's range", a.M, a.K);
}

template <int M, int R2>
int dispatch_ch(const W4Args &a, int ch, hipStream_t st) {
    constexpr int CHMAX = M <= 4 ? 4 : M <= 8 ? 2 : 1;
    if (ch == 1) return launch<M, R2, 1>(a, st);
    if constexpr (CHMAX >= 2) if (ch == 2) return launch<M, R2, 2>(a, st);
    if constexpr (CHMAX >= 4) {
        if (ch == 3) return launch<M, R2, 3>(a, st);
        if (ch == 4) return launch<M, R2, 4>(a, st);
    }
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w4a8: no kernel for M-tile %d with %d chunks", M, ch);
}

template <int M>
int dispatch_r(const W4Args &a, const Plan &p, hipStream_t st) {
    if (p.r2 == 1) return dispatch_ch<M, 1>(a, p.ch, st);
    if constexpr (4 * M <= 64) if (p.r2 == 2) return dispatch_ch<M, 2>(a, p.ch, st);
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w4a8: no kernel for %d row pairs", p.r2);
}

}  // namespace

namespace {

int run_gemv_w4a8(const char *who, const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs,
                  const void *xb, int8_t *xq_out, float *xs_out, void *y, int32_t *group_acc, int M, int N,
                  int K, int gs, void *stream) {
    CMI_REQUIRE(M >= 1 && M <= 16, CMI_E_UNSUPPORTED, "%s: M=%d outside 1..16", who, M);
    CMI_REQUIRE(gs == 64 || gs == 128 || gs == 256, CMI_E_UNSUPPORTED, "%s: group size %d, kernels are built for 64, 128 and 256", who, gs);
    CMI_REQUIRE(N >= 1 && K >= gs, CMI_E_ARG, "%s: bad shape N=%d K=%d", who, N, K);
    CMI_REQUIRE(K % gs == 0, CMI_E_UNSUPPORTED, "%s: K=%d is not a multiple of the group size %d (pad the rows with zeros)", who, K, gs);
    CMI_REQUIRE(gs == GS || !xb, CMI_E_UNSUPPORTED, "%s: group size %d takes quantised rows only", who, gs);
    const int lg = gs == 64 ? 1 : gs == 128 ? 2 : 3;
    const Plan p = make_plan(M, N, K, lg);
    W4Args a;
    a.w4 = w4;
    a.ws = ws;
    a.xq = xq;
    a.xs = xs;
    a.xb = static_cast<const uint16_t *>(xb);
    a.xq_out = xq_out;
    a.xs_out = xs_out;
    a.y = static_cast<uint16_t *>(y);
    a.group_acc = group_acc;
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = K / gs;
    a.nchunks = K / 32;
    a.KW = p.kw;
    a.teams = p.teams;
    a.iters = p.iters;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (lg != 2) {
        switch (p.mt) {
            case 1: return launch_other_group<1>(a, p.ch, lg, st);
            case 2: return launch_other_group<2>(a, p.ch, lg, st);
            case 4: return launch_other_group<4>(a, p.ch, lg, st);
            case 8: return launch_other_group<8>(a, p.ch, lg, st);
            default: return launch_other_group<16>(a, p.ch, lg, st);
        }
    }
    switch (p.mt) {
        case 1: return dispatch_r<1>(a, p, st);
        case 2: return dispatch_r<2>(a, p, st);
        case 4: return dispatch_r<4>(a, p, st);
        case 8: return dispatch_r<8>(a, p, st);
        default: return dispatch_r<16>(a, p, st);
    }
}

}  // namespace

extern "C" int cmi_gemv_w4a8(const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs,
                             void *y, int32_t *group_acc, int M, int N, int K, int gs,
                             void *stream) {
    CMI_REQUIRE(w4 && ws && xq && xs && y, CMI_E_ARG, "cmi_gemv_w4a8: null pointer");
    CMI_REQUIRE(aligned(w4, 16) && aligned(xq, 16), CMI_E_ARG,
                "cmi_gemv_w4a8: w4 and xq must be 16-byte aligned");
    if (gs == GS && N >= 1 && M >= 1) {
        // One row: the dot-product kernels.  The one that keeps the fp32 chain in registers takes any
        // K up to 20480 (5120 -> 25600: 13.0 us against 20.9 on the matrix-pipe kernel, 9728 -> 9728:
        // 11.6 against 23.2); without it (switched off, or longer rows) the older one while a
        // wavefront can hold its whole rows (K <= 4096) or the grid is small enough that the
        // wavefronts of a workgroup share rows.
        // Two rows: the same kernels only for whole rows of a large weight (2560 -> 151936: 34.5 us
        // against 42); otherwise, and from three rows, group sums on the matrix pipe.
        const bool chain_on = option_w4_decode_chain() != 1;
        const bool shared_rows = (N + 15) / 16 < 256, whole_rows = K <= (chain_on ? 5120 : 4096);
        const bool forced = option_w4_decode_chain() > 1 && M <= 2;  // a variant named by the caller
        int rc = CMI_E_UNSUPPORTED;
        if ((M == 1 && (whole_rows || shared_rows || (chain_on && K <= 20480))) ||
            (M == 2 && whole_rows && N >= 12288) || forced)
            rc = gemv_w4a8_decode(w4, ws, nullptr, xq, xs, y, group_acc, nullptr, nullptr, M, N, K, stream);
        if (rc == CMI_E_UNSUPPORTED)
            rc = gemv_w4a8_rows16(w4, ws, xq, xs, nullptr, y, group_acc, nullptr, nullptr, M, N, K, stream);
        if (rc == CMI_E_UNSUPPORTED && M <= 2)
            rc = gemv_w4a8_decode(w4, ws, nullptr, xq, xs, y, group_acc, nullptr, nullptr, M, N, K, stream);
        if (rc != CMI_E_UNSUPPORTED) return rc;
    }
    return run_gemv_w4a8("cmi_gemv_w4a8", w4, ws, xq, xs, nullptr, nullptr, nullptr, y, group_acc, M, N, K, gs,
                         stream);
}

extern "C" int cmi_gemv_w4a8_bf16(const uint8_t *w4, const float *ws, const void *x, void *y,
                                  int32_t *group_acc, int8_t *xq_out, float *xs_out, int M, int N, int K,
                                  int gs, void *stream) {
    CMI_REQUIRE(w4 && ws && x && y, CMI_E_ARG, "cmi_gemv_w4a8_bf16: null pointer");
    CMI_REQUIRE(aligned(w4, 16) && aligned(x, 16) && (!xq_out || aligned(xq_out, 8)), CMI_E_ARG,
                "cmi_gemv_w4a8_bf16: w4 and x must be 16-byte aligned, xq_out 8-byte aligned");
    CMI_REQUIRE(M >= 1 && M <= FUSED_MAX_ROWS, CMI_E_UNSUPPORTED,
                "cmi_gemv_w4a8_bf16: M=%d outside 1..%d (quantise with cmi_quant_act_i8 and call cmi_gemv_w4a8)",
                M, FUSED_MAX_ROWS);
    CMI_REQUIRE(N >= 1 && K >= GS, CMI_E_ARG, "cmi_gemv_w4a8_bf16: bad shape N=%d K=%d", N, K);
    CMI_REQUIRE(gs == GS, CMI_E_UNSUPPORTED, "cmi_gemv_w4a8_bf16: group size %d, the fused kernels are built for %d (quantise and call cmi_gemv_w4a8)", gs, GS);
    CMI_REQUIRE(K % GS == 0, CMI_E_UNSUPPORTED, "cmi_gemv_w4a8_bf16: K=%d is not a multiple of %d", K, GS);
    // long rows: the matrix-pipe kernel with the quantiser folded in (the dot-product kernel shares
    // such rows among wavefronts and its fp32 chain serialises: 10.5 us at 9728 -> 2560; or holds
    // 10-20 KiB per wavefront: 5120 -> 25600 42 us against 26); else the
    // decode kernel (whole rows requested up front) where it applies, else the general one
    int rc = CMI_E_UNSUPPORTED;
    // (one row of a weight whose grid is small enough that the wavefronts of a workgroup share
    // rows is the exception since that kernel's walk over the groups was made branch-free:
    // 9728 -> 2560 8.6 -> 8.25 us, 6144 -> 1024 5.9 -> 4.6 us)
    const bool one_shared_row = M == 1 && (N + 15) / 16 < 256;
    const int whole_row_k = option_w4_decode_chain() == 1 ? 4096 : 5120;
    if (K > whole_row_k && !one_shared_row && !(option_w4_decode_chain() > 1))
        rc = gemv_w4a8_rows16(w4, ws, nullptr, nullptr, x, y, group_acc, xq_out, xs_out, M, N, K, stream);
    if (rc != CMI_E_UNSUPPORTED) return rc;
    rc = gemv_w4a8_decode(w4, ws, x, nullptr, nullptr, y, group_acc, xq_out, xs_out, M, N, K, stream);
    if (rc != CMI_E_UNSUPPORTED) return rc;
    if (K > 4096 && one_shared_row)  // beyond the decode kernel's K
        rc = gemv_w4a8_rows16(w4, ws, nullptr, nullptr, x, y, group_acc, xq_out, xs_out, M, N, K, stream);
    if (rc != CMI_E_UNSUPPORTED) return rc;
    return run_gemv_w4a8("cmi_gemv_w4a8_bf16", w4, ws, nullptr, nullptr, x, xq_out, xs_out, y, group_acc, M, N, K,
                         gs, stream);
}
