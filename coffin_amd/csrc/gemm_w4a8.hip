// W4A8 prefill GEMM for CDNA4 int8 MFMA on the re-laid-out int4 weight (group size 128).
//
//   sum_g  = sum_{k in group g} xq[m,k] * (code(n,k) - 8)     int32, exact
//   total  = fma((float)sum_g, ws[n,g], total)                 g = 0,1,.. from 0.f
//   y[m,n] = bf16(total * xs[m])
//
// Same bits as the W4A8 GEMV for every m: the integer part is exact and the
// fp32 part is the one chain over the groups in ascending order.
//
// Block tile 128(m) x 128(n), 4 wavefronts (2 x 2) of 64 x 64, v_mfma_i32_32x32x32_i8,
// K walked one scale group (128) per step, two LDS stages, two workgroups per CU.
//   - activations go global -> LDS directly (global_load_lds_dwordx4, chunk
//     index XOR-swizzled on the global side, as in the W8A8 kernel);
//   - the packed weight (64 B per row and step) is fetched into registers one
//     step ahead, widened there to int8 code-8 (no cross-byte borrow), and
//     written to LDS once per workgroup, so the inner loop is the int8 one;
//   - the activation is the MFMA row operand and the weight the column operand:
//     a lane then owns ONE n per MFMA tile (and 16 m), so the per-group flush
//     total = fma((float)sum, ws[n,g], total) needs one scale per tile and lane,
//     fetched from memory a step ahead;
//   - the integer accumulators restart every step (first MFMA of a group takes
//     C = 0); the flush is 64 converts + 64 fmas per lane and step, which is why
//     two workgroups share a CU: one flushes while the other multiplies.
#include <cmath>
#include <cstdlib>

#include "common.hpp"
#include "gemm_tiles.hpp"

#include <type_traits>

namespace {

using namespace cmi;

constexpr int BM = 128, BN = 128, BK = 128;  // BK = the scale group
constexpr int THREADS = 256;
constexpr int X_BYTES = BM * BK, W_BYTES = BN * BK;  // int8 in LDS
constexpr int STAGE_BYTES = X_BYTES + W_BYTES;
constexpr int LDS_BYTES = 2 * STAGE_BYTES;           // 64 KiB

struct Args {
    const int8_t *xq;
    const uint8_t *w4;
    const float *xs;
    const float *ws;  // [N, G]
    uint16_t *y;
    int32_t *group_acc;  // [M, G, N], nullable
    int M, N, K, G;
    int ldy;  // row pitch of y (elements), >= N
    int tiles_m, tiles_n;
};

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// DUMP: also write the int32 group sums (parity checks); a separate instantiation, the
// 64 extra store addresses per lane would otherwise be carried through the hot loop.
// LG: log2(group size / 32).  2: a K step is a group (what the kernel is tuned for).  3: a group is
// two steps, the integer accumulators run on over the odd step and flush behind it.  1: a step holds
// two groups, flushed behind the second and the fourth k quarter.
template <bool DUMP, int LG = 2>
__global__ void __launch_bounds__(THREADS, 2)
gemm_w4a8_kernel(const Args a) {
    static_assert(LG >= 1 && LG <= 3, "group sizes 64, 128, 256");
    extern __shared__ __align__(16) int8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave & 1, wm = wave >> 1;

    // banded tile order per XCD (gemm_tiles.hpp)
    int tm, tn;
    banded_tile(a.tiles_m, a.tiles_n, blockIdx.x, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // activations: direct loads, wavefront w fills rows 32w..32w+31 (4 loads of 8 rows x 128 B)
    const int lrow = lane >> 3;
    const int8_t *xsrc[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int row = (4 * wave + g) * 8 + lrow;
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        xsrc[g] = a.xq + (size_t)min(m0 + row, a.M - 1) * a.K + kc * 16;
    }
    auto issue_x = [&](int stage, int ks) {
        int8_t *base = lds + stage * STAGE_BYTES + (4 * wave) * 1024;
#pragma unroll
        for (int g = 0; g < 4; ++g)
            __builtin_amdgcn_global_load_lds((const void *)(xsrc[g] + ks * BK), (lds_ptr_t)(base + g * 1024), 16, 0, 0);
    };

    // packed weight: 128 rows x 64 B per step = 512 x 16 B, two per thread; thread t takes
    // 16-byte piece (t%4) of rows t/4 and t/4 + 64.  A piece holds 32 k: LDS chunks 2p, 2p+1.
    const int wr = threadIdx.x >> 2, wp = threadIdx.x & 3;
    const uint8_t *wsrc[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
        wsrc[h] = a.w4 + (size_t)min(n0 + wr + 64 * h, a.N - 1) * (a.K / 2) + wp * 16;
    auto fetch_w = [&](uint4 (&reg)[2], int ks) {
#pragma unroll
        for (int h = 0; h < 2; ++h) reg[h] = *reinterpret_cast<const uint4 *>(wsrc[h] + ks * (BK / 2));
    };
    auto stash_w = [&](int stage, const uint4 (&reg)[2]) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int row = wr + 64 * h;
            const uint32_t w[4] = {reg[h].x, reg[h].y, reg[h].z, reg[h].w};
            uint4 lo, hi;  // k 0..15 and 16..31 of the piece
            widen_w4_piece(w[0], w[1], w[2], w[3], lo, hi);
            int8_t *dst = lds + stage * STAGE_BYTES + X_BYTES + row * BK;
            const int sw = (row >> 1) & 7;
            *reinterpret_cast<uint4 *>(dst + ((2 * wp) ^ sw) * 16) = lo;
            *reinterpret_cast<uint4 *>(dst + ((2 * wp + 1) ^ sw) * 16) = hi;
        }
    };

    // group scales of this lane's two n (one per MFMA column tile)
    const float *wsp[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
        wsp[j] = a.ws + (size_t)min(n0 + wn * 64 + j * 32 + (lane & 31), a.N - 1) * a.G;

    // fragments: lane reads row (lane%32) of a 32-row tile; k quarter q -> chunk 2q + lane/32
    const int frow = lane & 31;
    const int fsw = (frow >> 1) & 7;
    int foff[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) foff[q] = frow * BK + ((2 * q + (lane >> 5)) ^ fsw) * 16;
    struct Frag {
        v4i32 x[2], w[2];
    };
    auto read_q = [&](int stage, int q, Frag &f) {
        const int8_t *xt = lds + stage * STAGE_BYTES + wm * 64 * BK + foff[q];
        const int8_t *wt = lds + stage * STAGE_BYTES + X_BYTES + wn * 64 * BK + foff[q];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            f.x[t] = *reinterpret_cast<const v4i32 *>(xt + t * 32 * BK);
            f.w[t] = *reinterpret_cast<const v4i32 *>(wt + t * 32 * BK);
        }
    };

    float total[2][2][16];  // [m tile][n tile][element]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) total[i][j][v] = 0.f;

    const int ksteps = a.K / BK;
    const int mb = m0 + wm * 64, nb = n0 + wn * 64;
    v16i32 acc[2][2];
    auto mma_q = [&](const Frag &f, bool first) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (first) {
                    const v16i32 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.x[i], f.w[j], zero, 0, 0, 0);
                } else {
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.x[i], f.w[j], acc[i][j], 0, 0, 0);
                }
            }
    };

    // One group.  Its first-quarter fragments are in f0; stage ks%2 holds its operands.  After
    // the third quarter's reads the stage is free: the activations of step ks+1 have landed in
    // the other stage (requested a step ago), this wavefront's share of the weights of step
    // ks+1 (in registers since a step ago) is widened into it, and behind the barrier the
    // requests for step ks+2 go out while the last quarter multiplies.
    Frag f0, f1;
    uint4 wreg[2];
    float sc[2];
    float sc_b[2] = {0.f, 0.f};  // LG == 1: scales of the step's second group
    auto dump = [&](int group) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int n = nb + j * 32 + (lane & 31);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int m = mb + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                    if (m < a.M && n < a.N) a.group_acc[((size_t)m * a.G + group) * a.N + n] = acc[i][j][v];
                }
            }
    };
    auto flush = [&](const float (&scale)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) total[i][j][v] = fmaf((float)acc[i][j][v], scale[j], total[i][j][v]);
    };
    auto step = [&](auto more_tag, int ks) {
        constexpr bool MORE = decltype(more_tag)::value;  // a step ks+2 exists
        const int cur = ks & 1;
        const bool opens = LG == 3 ? (ks & 1) == 0 : true;   // this step starts a group
        const bool closes = LG == 3 ? (ks & 1) == 1 || ks + 1 == ksteps : true;
        // four MFMAs with the four fragment reads of the next quarter spread between them
        auto pace_quarter = [&]() {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
        };
        read_q(cur, 1, f1);
        mma_q(f0, opens);
        pace_quarter();
        read_q(cur, 2, f0);
        mma_q(f1, false);
        pace_quarter();
        if constexpr (LG == 1) {  // the step's first group is complete
            if constexpr (DUMP) dump(2 * ks);
            flush(sc);
        }
        read_q(cur, 3, f1);
        mma_q(f0, LG == 1);
        pace_quarter();
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        if (ks + 1 < ksteps) stash_w(cur ^ 1, wreg);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        float sc_next[2] = {0.f, 0.f}, sc_next_b[2] = {0.f, 0.f};
        if constexpr (MORE) {
            issue_x(cur, ks + 2);
            fetch_w(wreg, ks + 2);
        }
        if (ks + 1 < ksteps) {
            // scales of the group(s) the next step meets: group = step (LG 2), step / 2 (LG 3), 2 step and 2 step + 1 (LG 1)
            const int g = LG == 3 ? (ks + 1) >> 1 : LG == 1 ? 2 * (ks + 1) : ks + 1;
            sc_next[0] = wsp[0][g];
            sc_next[1] = wsp[1][g];
            if constexpr (LG == 1) {
                sc_next_b[0] = wsp[0][g + 1];
                sc_next_b[1] = wsp[1][g + 1];
            }
        }
        read_q(cur ^ 1, 0, f0);  // past the last step: a stale stage nobody uses
        mma_q(f1, false);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (MORE) __builtin_amdgcn_sched_group_barrier(0x010, 2, 0);  // requests for step ks+2
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        if (closes) {
            if constexpr (DUMP) dump(LG == 3 ? ks >> 1 : LG == 1 ? 2 * ks + 1 : ks);
            if constexpr (LG == 1) flush(sc_b);
            else flush(sc);
        }
        sc[0] = sc_next[0];
        sc[1] = sc_next[1];
        if constexpr (LG == 1) {
            sc_b[0] = sc_next_b[0];
            sc_b[1] = sc_next_b[1];
        }
    };
    using more_t = std::integral_constant<bool, true>;
    using last_t = std::integral_constant<bool, false>;

    // prologue: stage 0 complete (activations direct, weights through registers), step 1 on its way
    issue_x(0, 0);
    fetch_w(wreg, 0);
    sc[0] = wsp[0][0];
    sc[1] = wsp[1][0];
    if constexpr (LG == 1) {
        sc_b[0] = wsp[0][1];
        sc_b[1] = wsp[1][1];
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    stash_w(0, wreg);
    if (ksteps > 1) {
        issue_x(1, 1);
        fetch_w(wreg, 1);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_q(0, 0, f0);
    int ks = 0;
    for (; ks + 2 < ksteps; ++ks) step(more_t{}, ks);
    for (; ks < ksteps; ++ks) step(last_t{}, ks);

    // y[m,n] = bf16(total * xs[m]); a lane holds one n per tile: 32 lanes write 64 contiguous bytes
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int m = mb + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
            if (m >= a.M) continue;
            const float xm = a.xs[m];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int n = nb + j * 32 + (lane & 31);
                if (n < a.N) a.y[(size_t)m * a.ldy + n] = (uint16_t)f32_to_bf16_bits(total[i][j][v] * xm);
            }
        }
}

}  // namespace

static inline int a_ceil(int a, int b) { return (a + b - 1) / b; }

extern "C" int cmi_gemm_w4a8(const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs,
                             void *y, int32_t *group_acc, int M, int N, int K, int gs,
                             void *stream) {
    CMI_REQUIRE(M >= 0 && N >= 1 && K >= BK, CMI_E_ARG, "cmi_gemm_w4a8: bad shape M=%d N=%d K=%d", M, N, K);
    if (M == 0) return CMI_OK;  // an empty batch has no storage to point at
    CMI_REQUIRE(w4 && ws && xq && xs && y, CMI_E_ARG, "cmi_gemm_w4a8: null pointer");
    CMI_REQUIRE(gs == 64 || gs == BK || gs == 256, CMI_E_UNSUPPORTED,
                "cmi_gemm_w4a8: group size %d, kernels are built for 64, 128 and 256", gs);
    CMI_REQUIRE(K % BK == 0 && K % gs == 0, CMI_E_UNSUPPORTED,
                "cmi_gemm_w4a8: K=%d is not a multiple of 128 and of the group size %d (pad the rows with zeros)", K, gs);
    CMI_REQUIRE(aligned(xq, 16) && aligned(w4, 16), CMI_E_ARG,
                "cmi_gemm_w4a8: xq and w4 must be 16-byte aligned");
    // Which kernel: with few tiles a launch is a chain of K/128 dependent steps and the kernels differ
    // in the length of a step (two-stage 128 x 128 tiles: 1.15 us and up; ring of stages with
    // 64 x 64 tiles 0.44 us, with 128 x 64 tiles 0.6 us), with many tiles in how a step's time grows
    // with the tiles per CU, and up to 256 rows the matrix-pipe GEMV reads the weight once per 128
    // rows at memory speed and pays per 16-row chunk.  Same integer sums, same fp32 chain, same
    // bits from all of them.  Cost models (us) fitted to cold-weight measurements on ten layer
    // shapes x eleven batch sizes.  The ring kernels do not write the group sums.
    const int forced = option_gemm_tile();
    int ring = !group_acc && gs == BK && (forced == 64 || forced == 6464) ? forced : 0;
    // groups of 64 and 256: the two-stage tile kernel (and, up to 16 rows, the general GEMV)
    if (gs != BK && M <= 16 && !forced) return cmi_gemv_w4a8(w4, ws, xq, xs, y, group_acc, M, N, K, gs, stream);
    if (!forced && gs == BK) {
        const double steps = K / 128.0, wn = (double)N * K;
        const double tiles = (double)a_ceil(M, BM) * a_ceil(N, BN);
        const double t_tiled = 3.0 + steps * (tiles <= 512 ? 1.15 + 0.0013 * tiles : 1.6 * ceil(tiles / 512.0));
        // up to 10240 elements per row the GEMV keeps the weight in registers for 128 rows per launch
        // and pays per 16-row chunk only the chunk's sums and chain; longer rows run it in passes,
        // 16 rows per launch, at about half the speed
        const double t_rows16 =
            M > 256 ? 1e30
            : K <= 10240 ? a_ceil(M, 128) * (2.0 + wn / 2 / 4.2e6) + a_ceil(M, 16) * (0.6 + wn / 1.3e7 + steps * 0.012)
                         : a_ceil(M, 16) * (3.6 + wn / 2 / 2.1e6);
        const double tiles_h = (double)a_ceil(M, 64) * a_ceil(N, 64), tiles_g = (double)a_ceil(M, 128) * a_ceil(N, 64);
        // a step of the ring kernels: flat while every tile has a CU to itself, a second level up to
        // two tiles per CU, then linear in the tiles
        const double s_h = tiles_h <= 256 ? 0.44 + 6e-6 * N : tiles_h <= 512 ? 0.65 + 1e-5 * N : 0.4 + 0.00137 * tiles_h;
        const double s_g = tiles_g <= 256 ? 0.60 + 1.4e-5 * N : tiles_g <= 512 ? 1.0 + 4e-6 * N : 0.4 + 0.00205 * tiles_g;
        const double t_h = group_acc ? 1e30 : 2.5 + steps * s_h;
        const double t_g = group_acc ? 1e30 : 2.5 + steps * s_g;
        // (the GEMV's model is the optimistic one of the four at four chunks and more: it has to win by 10 %)
        if (t_rows16 <= t_tiled && t_rows16 <= 0.9 * t_h && t_rows16 <= 0.9 * t_g) {
            const int G = K / BK;
            const int step = K <= 10240 ? 128 : 16;
            for (int lo = 0; lo < M; lo += step) {
                const int m = M - lo < step ? M - lo : step;
                const int rc = gemv_w4a8_rows16(w4, ws, xq + (size_t)lo * K, xs + lo, nullptr,
                                                static_cast<uint16_t *>(y) + (size_t)lo * N,
                                                group_acc ? group_acc + (size_t)lo * G * N : nullptr, nullptr,
                                                nullptr, m, N, K, stream);
                if (rc != CMI_OK) return rc == CMI_E_UNSUPPORTED ? fail(rc, "cmi_gemm_w4a8: internal dispatch") : rc;
            }
            return CMI_OK;
        }
        if (t_h <= t_tiled && t_h <= t_g) ring = 6464;
        else if (t_g <= t_tiled) ring = 64;
    }
    if (ring) return gemm_w4a8_ring(w4, ws, xq, xs, y, M, N, K, ring, stream);
    Args a;
    a.xq = xq;
    a.w4 = w4;
    a.xs = xs;
    a.ws = ws;
    a.y = static_cast<uint16_t *>(y);
    a.group_acc = group_acc;
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = K / gs;
    a.ldy = N;
    a.tiles_m = (M + BM - 1) / BM;
    a.tiles_n = (N + BN - 1) / BN;
    // Whole rounds.  Two workgroups share a CU, so a launch runs in rounds of 512 tiles and a last
    // round that is nearly empty costs as much as a full one (1024 x 25600: 1600 tiles = 3.125
    // rounds, 252 us against 211 us for the 3.000 rounds of N = 24576).  The n tiles of such a
    // remainder (at most half a round) go to a second launch of 64 x 64 tiles with a ring of
    // stages, whose step is 0.44 us instead of 1.15 us and which spreads them over all CUs:
    // same arithmetic, same bits.  (Not when the group sums are asked for: the ring kernels do not
    // write them.)
    int ring_n = 0;  // columns handed to the second launch
    if (!forced && gs == BK && !group_acc) {
        const int slots = 512, tiles = a.tiles_m * a.tiles_n, rest = tiles % slots;
        if (tiles > slots && rest > 0 && rest <= slots / 2 && rest % a.tiles_m == 0) {
            const int rest_n = rest / a.tiles_m;             // n tiles of the remainder
            const int cols = N - (a.tiles_n - rest_n) * BN;  // their columns (the last tile may be ragged)
            const double steps = K / 128.0, tiles_h = (double)a_ceil(M, 64) * a_ceil(cols, 64);
            const double s_h = tiles_h <= 256 ? 0.44 + 6e-6 * cols : tiles_h <= 512 ? 0.65 + 1e-5 * cols : 0.4 + 0.00137 * tiles_h;
            if (2.5 + steps * s_h < steps * 1.15) {
                ring_n = cols;
                a.N = N - cols;
                a.tiles_n -= rest_n;
            }
        }
    }
    const dim3 grid(a.tiles_m * a.tiles_n), block(THREADS);
    hipStream_t st = static_cast<hipStream_t>(stream);
    static std::atomic<uint64_t> devices[6];
    auto run = [&](auto kernel, int slot) {
        if (const int rc = reserve_lds(reinterpret_cast<const void *>(kernel), LDS_BYTES, devices[slot], "cmi_gemm_w4a8"))
            return rc;
        kernel<<<grid, block, LDS_BYTES, st>>>(a);
        return check_launch("cmi_gemm_w4a8");
    };
    if (gs == 64) return group_acc ? run(gemm_w4a8_kernel<true, 1>, 0) : run(gemm_w4a8_kernel<false, 1>, 1);
    if (gs == 256) return group_acc ? run(gemm_w4a8_kernel<true, 3>, 2) : run(gemm_w4a8_kernel<false, 3>, 3);
    if (const int rc = group_acc ? run(gemm_w4a8_kernel<true, 2>, 4) : run(gemm_w4a8_kernel<false, 2>, 5)) return rc;
    if (!ring_n) return CMI_OK;
    const int n1 = N - ring_n;
    return gemm_w4a8_ring(w4 + (size_t)n1 * (K / 2), ws + (size_t)n1 * a.G, xq, xs, static_cast<uint16_t *>(y) + n1, M, ring_n,
                          K, 6464, stream, N);
}
