// W4A8 GEMM with a ring of LDS stages, for launches of few tiles (batches of 17..256 rows, or
// few n tiles): same arithmetic and bits as gemm_w4a8.hip,
//
//   sum_g  = sum_{k in group g} xq[m,k] * (code(n,k) - 8)     int32, exact
//   total  = fma((float)sum_g, ws[n,g], total)                 g = 0,1,.. from 0.f
//   y[m,n] = bf16(total * xs[m])
//
// but built for the case where a launch is a chain of K / 128 dependent steps rather than a
// stream of MFMAs.  The two-stage kernel asks for the operands of a step one step ahead and
// waits for all of them every step; with a tile or fewer per CU a step then lasts as long as a
// trip to memory (1.2-1.4 us).  Here NST steps of operands are in flight:
//   - activations, the packed weight (64 B per row and step) and the group scales of a step all
//     go global -> LDS directly into the step's ring slot (no destination registers, so the
//     only waits are the explicit vmcnt counts);
//   - the lane that requested a 16-byte piece of packed weight reads it back from the slot when
//     it has landed (its own vmcnt: no barrier), widens it to int8 code-8 and writes it into one
//     of two int8 weight buffers, from which the four wavefronts take MFMA fragments;
//   - every wavefront requests the step's scales itself (one 4-byte direct load per 64 rows),
//     so the scales it reads are covered by its own vmcnt as well.
// Block tile (64 TM) x (64 TN), four wavefronts (2 x 2), v_mfma_i32_32x32x32_i8 with the
// activation as the row operand: a lane owns one n per MFMA tile and the per-group flush needs
// one scale per tile.  One barrier per step; a step's fragments are all read right behind it.
#include "common.hpp"
#include "gemm_tiles.hpp"

#include <type_traits>

namespace {

using namespace cmi;

constexpr int BK = 128;  // one scale group per step
constexpr int THREADS = 256;

struct Args {
    const int8_t *xq;
    const uint8_t *w4;
    const float *xs;
    const float *ws;  // [N, G]
    uint16_t *y;
    int M, N, K, G;
    int ldy;  // row pitch of y (elements), >= N
    int tiles_m, tiles_n;
};

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// LDS reads of what this lane's own direct loads have written, and the LDS writes of the widened
// weight.  The compiler keeps track of direct loads as LDS writes and puts a wait for ALL of them
// (vmcnt(0)) in front of an ordinary LDS read of the same region and of any ordinary LDS write,
// which would drain the ring at every step; the explicit vmcnt counts of the kernel are the
// synchronisation, so these accesses are issued where the compiler does not see them.
__device__ __forceinline__ uint32_t lds_offset(const void *p) {
    return (uint32_t)(uintptr_t)(lds_ptr_t)p;
}
__device__ __forceinline__ v4i32 lds_read16_unseen(const void *p) {
    v4i32 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(lds_offset(p)) : "memory");
    return v;
}
__device__ __forceinline__ float lds_read4_unseen(const void *p) {
    float v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(lds_offset(p)) : "memory");
    return v;
}

__device__ __forceinline__ void lds_write16_unseen(void *p, uint4 v) {
    const v4i32 d = {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
    asm volatile("ds_write_b128 %0, %1" ::"v"(lds_offset(p)), "v"(d) : "memory");
}

template <int TN, int TM, int NST>
struct Cfg {
    static constexpr int BN = 64 * TN, BM = 64 * TM;
    static constexpr int X_BYTES = BM * BK;      // int8 activations of a step
    static constexpr int P_BYTES = BN * BK / 2;  // packed weight of a step
    static constexpr int S_BYTES = BN * 4;       // group scales of a step
    static constexpr int SLOT_BYTES = X_BYTES + P_BYTES + S_BYTES;
    static constexpr int W_BYTES = BN * BK;      // widened weight, two buffers
    static constexpr int XS_OFF = NST * SLOT_BYTES + 2 * W_BYTES;  // row scales of the tile
    static constexpr int LDS_BYTES = XS_OFF + BM * 4;
    static constexpr int XL = BM / 32;           // activation loads per wavefront and step (8 rows each)
    static constexpr int LOADS = XL + 2 * TN;    // + packed weight (16 rows each) + scales (64 each)
    static_assert((NST - 1) * LOADS <= 63, "vmcnt range");
};

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    if constexpr (N == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if constexpr (N == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else if constexpr (N == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else if constexpr (N == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if constexpr (N == 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else if constexpr (N == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if constexpr (N == 18) asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
    else if constexpr (N == 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else static_assert(N < 0, "add the vmcnt literal");
}

template <int TN, int TM, int NST>
__global__ void __launch_bounds__(THREADS)
gemm_w4a8_ring_kernel(const Args a) {
    using C = Cfg<TN, TM, NST>;
    extern __shared__ __align__(16) int8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave & 1, wm = wave >> 1;

    // banded tile order per XCD (gemm_tiles.hpp)
    int tm, tn;
    banded_tile(a.tiles_m, a.tiles_n, blockIdx.x, tm, tn);
    const int m0 = tm * C::BM, n0 = tn * C::BN;

    // the tile's row scales, for the epilogue (read behind the loop's barriers)
    float *xs_tile = reinterpret_cast<float *>(lds + C::XS_OFF);
    for (int i = threadIdx.x; i < C::BM; i += THREADS) xs_tile[i] = a.xs[min(m0 + i, a.M - 1)];

    // Global side of the direct loads of one step.  Activations: 8 rows x 128 B per load, chunk
    // index XOR-swizzled by (row / 2) % 8; wavefront w fills rows 8 XL w .. 8 XL (w+1) - 1.
    // Packed weight: 16 rows x 64 B per load, lane l = piece l%4 of row l/4, unswizzled (only the
    // requesting lane reads it back).  Scales: 64 rows per load, every wavefront all of them.
    const int8_t *xsrc[C::XL];
#pragma unroll
    for (int g = 0; g < C::XL; ++g) {
        const int row = (C::XL * wave + g) * 8 + (lane >> 3);
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        xsrc[g] = a.xq + (size_t)min(m0 + row, a.M - 1) * a.K + kc * 16;
    }
    const uint8_t *psrc[TN];
#pragma unroll
    for (int h = 0; h < TN; ++h) {
        const int row = (TN * wave + h) * 16 + (lane >> 2);
        psrc[h] = a.w4 + (size_t)min(n0 + row, a.N - 1) * (a.K / 2) + (lane & 3) * 16;
    }
    const float *ssrc[TN];
#pragma unroll
    for (int h = 0; h < TN; ++h) ssrc[h] = a.ws + (size_t)min(n0 + 64 * h + lane, a.N - 1) * a.G;

    auto issue = [&](int slot, int ks) {
        int8_t *base = lds + slot * C::SLOT_BYTES;
#pragma unroll
        for (int g = 0; g < C::XL; ++g)
            __builtin_amdgcn_global_load_lds((const void *)(xsrc[g] + ks * BK),
                                             (lds_ptr_t)(base + (C::XL * wave + g) * 1024), 16, 0, 0);
#pragma unroll
        for (int h = 0; h < TN; ++h)
            __builtin_amdgcn_global_load_lds((const void *)(psrc[h] + ks * (BK / 2)),
                                             (lds_ptr_t)(base + C::X_BYTES + (TN * wave + h) * 1024), 16, 0, 0);
#pragma unroll
        for (int h = 0; h < TN; ++h)
            __builtin_amdgcn_global_load_lds((const void *)(ssrc[h] + ks),
                                             (lds_ptr_t)(base + C::X_BYTES + C::P_BYTES + h * 256), 4, 0, 0);
    };

    // This lane's pieces of packed weight, slot -> int8 buffer `buf` (chunks 2p, 2p+1 of the row,
    // swizzled like the activations), and the slot's scales of this lane's n.
    struct Fetched {
        v4i32 packed[TN];
        float sc[TN];
    };
    auto fetch = [&](int slot) {  // requests only
        const int8_t *src = lds + slot * C::SLOT_BYTES + C::X_BYTES;
        const float *s = reinterpret_cast<const float *>(src + C::P_BYTES);
        Fetched f;
#pragma unroll
        for (int h = 0; h < TN; ++h) f.packed[h] = lds_read16_unseen(src + (TN * wave + h) * 1024 + lane * 16);
#pragma unroll
        for (int j = 0; j < TN; ++j) f.sc[j] = lds_read4_unseen(s + wn * 32 * TN + j * 32 + (lane & 31));
        return f;
    };
    auto widen = [&](Fetched &f, int buf, float (&sc_out)[TN]) {
        int8_t *wbuf = lds + NST * C::SLOT_BYTES + buf * C::W_BYTES;
        if constexpr (TN == 1) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.packed[0]), "+v"(f.sc[0])::"memory");
        else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.packed[0]), "+v"(f.packed[1]), "+v"(f.sc[0]), "+v"(f.sc[1])::"memory");
        static_assert(TN <= 2, "operands of the wait above");
#pragma unroll
        for (int j = 0; j < TN; ++j) sc_out[j] = f.sc[j];
#pragma unroll
        for (int h = 0; h < TN; ++h) {
            const int row = (TN * wave + h) * 16 + (lane >> 2), wp = lane & 3;
            const uint32_t w[4] = {(uint32_t)f.packed[h].x, (uint32_t)f.packed[h].y, (uint32_t)f.packed[h].z,
                                   (uint32_t)f.packed[h].w};
            uint4 lo, hi;  // k 0..15 and 16..31 of the piece
            widen_w4_piece(w[0], w[1], w[2], w[3], lo, hi);
            int8_t *dst = wbuf + row * BK;
            const int sw = (row >> 1) & 7;
            lds_write16_unseen(dst + ((2 * wp) ^ sw) * 16, lo);
            lds_write16_unseen(dst + ((2 * wp + 1) ^ sw) * 16, hi);
        }
    };

    // fragments: lane reads row (lane%32) of a 32-row tile; k quarter q -> chunk 2q + lane/32
    const int frow = lane & 31;
    const int fsw = (frow >> 1) & 7;
    int foff[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) foff[q] = frow * BK + ((2 * q + (lane >> 5)) ^ fsw) * 16;
    struct Frag {
        v4i32 x[TM], w[TN];
    };
    auto read_q = [&](int slot, int buf, int q, Frag &f) {
        const int8_t *xt = lds + slot * C::SLOT_BYTES + wm * 32 * TM * BK + foff[q];
        const int8_t *wt = lds + NST * C::SLOT_BYTES + buf * C::W_BYTES + wn * 32 * TN * BK + foff[q];
#pragma unroll
        for (int t = 0; t < TM; ++t) f.x[t] = *reinterpret_cast<const v4i32 *>(xt + t * 32 * BK);
#pragma unroll
        for (int t = 0; t < TN; ++t) f.w[t] = *reinterpret_cast<const v4i32 *>(wt + t * 32 * BK);
    };
    float total[TM][TN][16];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) total[i][j][v] = 0.f;

    v16i32 acc[TM][TN];
    auto mma_q = [&](const Frag &f, bool first) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (first) {
                    const v16i32 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.x[i], f.w[j], zero, 0, 0, 0);
                } else {
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.x[i], f.w[j], acc[i][j], 0, 0, 0);
                }
            }
    };
    const int ksteps = a.K / BK;
    // Step ks enters with all its fragments in registers (read behind the previous barrier, under
    // the previous step's flush) and its scales in sc.  Its MFMAs go out back to back; this lane's
    // share of the next step's weight -- landed long ago (measured: the vmcnt wait is over before
    // it starts), asked for at the top of the step -- is widened into the other int8 buffer, which
    // step ks-1 has finished reading.  Behind the barrier slot ks % NST is free and takes the
    // requests of step ks+NST, the next step's fragments are requested, and the group sums are
    // flushed into the fp32 totals while they arrive.  No branches inside a step (past the last
    // step stale bytes are widened and read where nobody uses them).  Reading a quarter's fragments
    // under the previous quarter's MFMAs, as the W8A8 kernels do, left every LDS latency exposed
    // here (one MFMA per quarter and wavefront): 0.50 -> 0.44 us per step.
    Frag f[4];
    float sc[TN];
    auto step = [&](auto issue_tag, int ks) {
        constexpr bool ISSUE = decltype(issue_tag)::value;
        const int slot = ks % NST, next = (ks + 1) % NST, buf = ks & 1;
        if constexpr (ISSUE) wait_vmcnt<(NST - 2) * C::LOADS>();
        else wait_vmcnt<0>();
        Fetched fetched = fetch(next);
        mma_q(f[0], true);
        mma_q(f[1], false);
        mma_q(f[2], false);
        mma_q(f[3], false);
        float sc_next[TN];
        widen(fetched, buf ^ 1, sc_next);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if constexpr (ISSUE) issue(slot, ks + NST);
#pragma unroll
        for (int q = 0; q < 4; ++q) read_q(next, buf ^ 1, q, f[q]);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) total[i][j][v] = fmaf((float)acc[i][j][v], sc[j], total[i][j][v]);
#pragma unroll
        for (int j = 0; j < TN; ++j) sc[j] = sc_next[j];
    };
    using issue_t = std::integral_constant<bool, true>;
    using drain_t = std::integral_constant<bool, false>;

    for (int s = 0; s < NST; ++s)
        if (s < ksteps) issue(s, s);
    if (ksteps >= NST) wait_vmcnt<(NST - 1) * C::LOADS>();
    else wait_vmcnt<0>();
    {
        Fetched first = fetch(0);
        widen(first, 0, sc);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int q = 0; q < 4; ++q) read_q(0, 0, q, f[q]);
    const int n_issue = ksteps > NST ? ksteps - NST : 0;
    int ks = 0;
    for (; ks < n_issue; ++ks) step(issue_t{}, ks);
    for (; ks < ksteps; ++ks) step(drain_t{}, ks);

    // y[m,n] = bf16(total * xs[m]); a lane holds one n per tile: 32 lanes write 64 contiguous bytes
    const int mb = wm * 32 * TM, nb = n0 + wn * 32 * TN;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int ml = mb + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
            const int m = m0 + ml;
            if (m >= a.M) continue;
            const float xm = xs_tile[ml];
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = nb + j * 32 + (lane & 31);
                if (n < a.N) a.y[(size_t)m * a.ldy + n] = (uint16_t)f32_to_bf16_bits(total[i][j][v] * xm);
            }
        }
}

template <int TN, int TM, int NST>
int launch(Args &a, hipStream_t st) {
    using C = Cfg<TN, TM, NST>;
    a.tiles_m = (a.M + C::BM - 1) / C::BM;
    a.tiles_n = (a.N + C::BN - 1) / C::BN;
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemm_w4a8_ring_kernel<TN, TM, NST>),
                                   C::LDS_BYTES, devices, "cmi_gemm_w4a8"))
        return rc;
    gemm_w4a8_ring_kernel<TN, TM, NST><<<dim3(a.tiles_m * a.tiles_n), dim3(THREADS), C::LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemm_w4a8");
}

}  // namespace

namespace cmi {

// tile: 6464 (64 x 64) or 64 (128 m x 64 n); with 128 x 128 tiles the ring measured no faster than
// the two-stage kernel, two of whose workgroups share a CU.  Arguments already checked by the
// caller (K % 128 == 0, group size 128, 16-byte aligned xq and w4).
int gemm_w4a8_ring(const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs, void *y, int M, int N,
                   int K, int tile, void *stream, int ldy) {
    Args a;
    a.xq = xq;
    a.w4 = w4;
    a.xs = xs;
    a.ws = ws;
    a.y = static_cast<uint16_t *>(y);
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = K / BK;
    a.ldy = ldy > 0 ? ldy : N;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (tile == 6464) return launch<1, 1, 4>(a, st);
    if (tile == 64) return launch<1, 2, 3>(a, st);
    return CMI_E_UNSUPPORTED;
}

}  // namespace cmi
