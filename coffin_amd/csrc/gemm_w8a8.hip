// W8A8 prefill GEMM for CDNA4 int8 MFMA (K a multiple of 128).
//
//   acc[m,n] = sum_k xq[m,k] * wq[n,k]           int32, exact
//   y[m,n]   = bf16((float)acc * xs[m] * ws[n])   left to right, one narrowing
//
// v_mfma_i32_32x32x32_i8 with the weight on the MFMA rows and the activation on
// the MFMA columns, both K-contiguous in memory (16 consecutive k per lane), so
// a lane ends with groups of four consecutive n of one m.
//
// Common to both kernels below: K is walked in steps of 128 (one whole cache
// line per row and request: with 64-byte steps every line is fetched from L2
// twice); operand tiles go global -> LDS directly (global_load_lds_dwordx4, no
// staging registers).  A direct load lays the 64 lanes' 16-byte chunks out
// contiguously, so the bank-conflict-free arrangement is made on the global
// side: lane i of a load fetches the chunk that belongs at LDS slot i, with the
// chunk index XOR-swizzled by (row / 2) % 8.  Waits are explicit vmcnt/lgkmcnt
// counts with one s_barrier per step (a __syncthreads would drain the prefetch),
// and the interleaving of MFMAs, LDS reads and global loads inside a step is
// spelled out with scheduling group barriers: left alone, the compiler puts the
// wait for the *next* fragments in front of the current MFMAs.  The epilogue goes
// through LDS once more so that every lane stores 16 contiguous bytes of y.
// Workgroup ids are remapped so each of the 8 XCDs (private L2) owns a
// contiguous band of n tiles.
//
//   gemm_w8a8_pipe_kernel: 128 x 128 block tile, 4 wavefronts of 64 x 64, two
//     LDS stages, whole-step fragment double buffering in registers, two
//     workgroups per CU (one's prologue/epilogue hides under the other's MFMAs).
//   gemm_w8a8_big_kernel: 256 x 256 block tile, 8 wavefronts of 128 x 64, a ring
//     of five single-operand LDS slots.  Half the L2 -> LDS bytes per MFMA.
//   gemm_w8a8_wide_kernel: 256 x 320 block tile, 8 wavefronts of 64 x 160, two LDS
//     stages; for shapes whose n extent tiles better by 320 (9728 = 30.4 x 320).
//
// The launcher picks by how well the tile count fills the 256 CUs.
#include "common.hpp"
#include "gemm_tiles.hpp"

#include <cmath>
#include <cstdlib>
#include <type_traits>

namespace {

using namespace cmi;

constexpr int BK = 128;        // one 128-byte cache line per row and step
constexpr double SPLIT128_HANDOVER_US = 11.0;  // split-K on 128 x 128 tiles: partials out, arrival, partials in (measured 10..11.5)
constexpr int THREADS = 256;   // 2 x 2 wavefronts

struct Args {
    const int8_t *xq;
    const int8_t *wq;
    const float *xs;
    const float *ws;
    uint16_t *y;
    int32_t *acc_out;
    int M, N, K, ldy;
    int tiles_m, tiles_n;
    // split-K launches only: how many workgroups share a tile's K range, where they leave their
    // int32 partial tiles ([split][tile][accumulator piece][thread] x 16 bytes) and the tiles'
    // arrival counters (zero at launch)
    int splits;
    int32_t *partials;
    int *arrivals;
    // pipe kernel: workgroups launched beyond the tiles (x splits), on CUs the tiles leave idle;
    // they read the weight through the caches (warm_caches in gemm_tiles.hpp)
    int warm_blocks;
};

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// TN, TM: 32 x 32 MFMA tiles per wavefront along n (weight rows) and m
// (activation rows); block tile = (64*TM) x (64*TN).  NST: LDS stages.
template <int TN, int TM, int NST>
struct Cfg {
    static constexpr int BN = 64 * TN, BM = 64 * TM;
    static constexpr int W_BYTES = BN * BK, X_BYTES = BM * BK;
    static constexpr int STAGE_BYTES = W_BYTES + X_BYTES;
    static constexpr int SCALE_BYTES = 4 * (BN + BM);   // the tile's scales, behind the stages
    static constexpr int LDS_BYTES = NST * STAGE_BYTES + SCALE_BYTES;
    static constexpr int WL = BN / 32, XL = BM / 32;  // loads per wavefront and stage (8 rows each)
    static constexpr int LPW = WL + XL;
    static constexpr int PITCH = 64 * TN + 16;        // epilogue: one m row of the wavefront tile + 16 B
    static_assert(4 * 32 * TM * PITCH <= NST * STAGE_BYTES, "epilogue does not fit the operand stages");
    static_assert((NST - 2) * LPW <= 63, "vmcnt range");
};

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    if constexpr (N == 0) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 3) asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 4) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 6) asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 8) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 9) asm volatile("s_waitcnt vmcnt(9) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 10) asm volatile("s_waitcnt vmcnt(10) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 12) asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 16) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 18) asm volatile("s_waitcnt vmcnt(18) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 20) asm volatile("s_waitcnt vmcnt(20) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 24) asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 28) asm volatile("s_waitcnt vmcnt(28) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 30) asm volatile("s_waitcnt vmcnt(30) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 32) asm volatile("s_waitcnt vmcnt(32) lgkmcnt(0)" ::: "memory");
    else if constexpr (N == 36) asm volatile("s_waitcnt vmcnt(36) lgkmcnt(0)" ::: "memory");
    else static_assert(N < 0, "add the vmcnt literal");
}

// Tile of this workgroup (the XCD-banded order of gemm_tiles.hpp).
__device__ __forceinline__ void tile_coords(const Args &a, int &tm, int &tn, int id = blockIdx.x) {
    banded_tile(a.tiles_m, a.tiles_n, id, tm, tn);
}

// Scales of a BN x BM block tile into LDS at `dst` (BN column scales, then BM row scales), indices
// clamped to the matrix; read again only behind the barrier that opens the epilogue.
template <int BN, int BM>
__device__ __forceinline__ void stage_scales(const Args &a, float *dst, int n0, int m0) {
    for (int i = threadIdx.x; i < BN + BM; i += blockDim.x)
        dst[i] = i < BN ? a.ws[min(n0 + i, a.N - 1)] : a.xs[min(m0 + i - BN, a.M - 1)];
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));

// Two fp32 -> packed bf16, round to nearest even (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2v));
}

// Epilogue of one wavefront tile of TN x TM MFMA tiles whose corner is (nb, mb).
// Accumulator element v of tile (i, j) in lane l is
//   n = nb + 32*i + 8*(v/4) + 4*(l/32) + v%4,   m = mb + 32*j + l%32.
// Scale, narrow, park the wavefront's bf16 tile in LDS (row = m), then write
// rows back 16 bytes per lane.  Every wavefront of the workgroup must call it
// (one barrier inside: the operand stages are reused as parking space).
// JP: m tiles parked per pass (the parking space of a wavefront is 32*JP rows); TM % JP == 0.
// ws_tile / xs_tile (nullable): the scales of the block tile staged in LDS by the kernel's prologue,
// indexed from the wavefront tile's corner (ws_tile[0] is ws[nb], xs_tile[0] is xs[mb]); fetched from
// global memory here they are cold loads at the head of the epilogue.
template <int TN, int TM, int JP = TM>
__device__ __forceinline__ void epilogue(const Args &a, v16i32 (&acc)[TN][TM], int8_t *lds, int wave,
                                         int lane, int nb, int mb, const float *ws_tile = nullptr,
                                         const float *xs_tile = nullptr) {
    if (a.acc_out) {
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const int m = mb + j * 32 + (lane & 31);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int n = nb + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                    if (m < a.M && n < a.N) a.acc_out[(size_t)m * a.N + n] = acc[i][j][v];
                }
            }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();  // every wavefront is done reading operand stages
    asm volatile("" ::: "memory");
    constexpr int PITCH = 64 * TN + 16;  // one m row of the wavefront tile + 16 B
    int8_t *park = lds + wave * (32 * JP * PITCH);
    // per-column scales of this lane's columns: 4 consecutive n per (i, q)
    float wsv[TN][4][4];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int n = nb + i * 32 + 8 * q + 4 * (lane >> 5);
            if (ws_tile) {
                const float4 sc = *reinterpret_cast<const float4 *>(ws_tile + (n - nb));
                wsv[i][q][0] = sc.x, wsv[i][q][1] = sc.y, wsv[i][q][2] = sc.z, wsv[i][q][3] = sc.w;
            } else if (n + 3 < a.N) {
                const float4 sc = *reinterpret_cast<const float4 *>(a.ws + n);
                wsv[i][q][0] = sc.x, wsv[i][q][1] = sc.y, wsv[i][q][2] = sc.z, wsv[i][q][3] = sc.w;
            } else {
                // ragged edge: clamped reads; those columns are never stored
#pragma unroll
                for (int r = 0; r < 4; ++r) wsv[i][q][r] = a.ws[min(n + r, a.N - 1)];
            }
        }
    const bool vec_ok = (a.ldy % 8 == 0) && ((reinterpret_cast<uintptr_t>(a.y) & 15) == 0);
    constexpr int CPR = 4 * TN;  // 16-byte chunks per row of the wavefront tile
#pragma unroll
    for (int j0 = 0; j0 < TM; j0 += JP) {
#pragma unroll
        for (int jj = 0; jj < JP; ++jj) {
            const int j = j0 + jj;
            const int ml = jj * 32 + (lane & 31);
            const float xm = xs_tile ? xs_tile[j * 32 + (lane & 31)] : a.xs[min(mb + j * 32 + (lane & 31), a.M - 1)];
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = i * 32 + 8 * q + 4 * (lane >> 5);
                    float t[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) t[r] = ((float)acc[i][j][4 * q + r] * xm) * wsv[i][q][r];
                    uint2 pk;
                    pk.x = pack_bf16(t[0], t[1]);
                    pk.y = pack_bf16(t[2], t[3]);
                    *reinterpret_cast<uint2 *>(park + ml * PITCH + nl * 2) = pk;
                }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own tile only: no barrier needed
        // RPI whole rows per iteration: lane -> (row r0, chunk c) once, then only
        // the row advances, so LDS offsets are immediates and the global
        // pointer moves by a fixed stride.
        constexpr int RPI = 64 / CPR;
        const int r0 = lane / CPR, c = lane - r0 * CPR;
        const int n = nb + c * 8;
        const bool lane_ok = r0 < RPI && n < a.N;
        const bool whole = vec_ok && n + 7 < a.N;
        const int8_t *src = park + r0 * PITCH + c * 16;
        int m = mb + j0 * 32 + r0;
        uint16_t *dst = a.y + (size_t)m * a.ldy + n;
        const size_t dstep = (size_t)RPI * a.ldy;
#pragma unroll
        for (int it = 0; it < (32 * JP + RPI - 1) / RPI; ++it, m += RPI, dst += dstep) {
            if (!lane_ok || m >= a.M || (it * RPI + RPI > 32 * JP && it * RPI + r0 >= 32 * JP)) continue;
            const uint4 v = *reinterpret_cast<const uint4 *>(src + it * RPI * PITCH);
            if (whole) {
                *reinterpret_cast<uint4 *>(dst) = v;
            } else {
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int r = 0; r < 8; ++r)
                    if (n + r < a.N) dst[r] = (uint16_t)(w[r >> 1] >> ((r & 1) * 16));
            }
        }
        if (j0 + JP < TM) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // reads done before the next pass parks
    }
}

// SPLIT: a.splits workgroups share a tile, each walking a contiguous part of K; they leave their
// int32 accumulators in a.partials and the last to arrive (a.arrivals, cleared before the launch)
// adds the others' to its own -- integer sums, exact in any order -- and runs the epilogue: the
// bits of the unsplit kernel.  For launches of few tiles and many K steps, which are a chain of
// dependent steps on a fraction of the CUs.
template <int TN, int TM, int NST, bool SPLIT = false>
__global__ void __launch_bounds__(THREADS)
gemm_w8a8_pipe_kernel(const Args a) {
    using C = Cfg<TN, TM, NST>;
    extern __shared__ __align__(16) int8_t lds[];
    __shared__ int arrived_before;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: keeps LDS bases scalar
    const int wn = wave & 1, wm = wave >> 1;

    const int tiles = a.tiles_m * a.tiles_n;
    const int work = SPLIT ? tiles * a.splits : tiles;
    if ((int)blockIdx.x >= work) {  // uniform: no tile, and before any barrier
        warm_caches(a.wq, (size_t)a.N * a.K, blockIdx.x - work, a.warm_blocks);
        return;
    }
    const int tile = SPLIT ? blockIdx.x % tiles : blockIdx.x, split = SPLIT ? blockIdx.x / tiles : 0;
    int tm, tn;
    tile_coords(a, tm, tn, tile);
    const int m0 = tm * C::BM, n0 = tn * C::BN;
    float *scales = reinterpret_cast<float *>(lds + NST * C::STAGE_BYTES);
    stage_scales<C::BN, C::BM>(a, scales, n0, m0);
    // this workgroup's K steps: all of them, or part `split` of a.splits nearly equal parts
    const int ksteps_all = a.K / BK;
    const int k_first = SPLIT ? (int)((long long)ksteps_all * split / a.splits) : 0;
    const int ksteps = SPLIT ? (int)((long long)ksteps_all * (split + 1) / a.splits) - k_first : ksteps_all;

    // Global side of the direct loads.  One load instruction moves 8 rows x 128 B
    // (whole cache lines) into 1 KiB of LDS; each wavefront fills a contiguous run
    // of rows (consecutive loads on consecutive rows measured 30 % faster than
    // wavefronts interleaved row group by row group).  Lane i lands in slot i of the group: row = i/8, stored chunk
    // = i%8, which holds k chunk (i%8) ^ ((row/2) % 8).
    const int lrow = lane >> 3;
    const int8_t *wsrc[C::WL], *xsrc[C::XL];
#pragma unroll
    for (int g = 0; g < C::WL; ++g) {
        const int row = (C::WL * wave + g) * 8 + lrow;
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        wsrc[g] = a.wq + (size_t)min(n0 + row, a.N - 1) * a.K + kc * 16 + k_first * BK;
    }
#pragma unroll
    for (int g = 0; g < C::XL; ++g) {
        const int row = (C::XL * wave + g) * 8 + lrow;
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        xsrc[g] = a.xq + (size_t)min(m0 + row, a.M - 1) * a.K + kc * 16 + k_first * BK;
    }
    auto issue = [&](int stage, int ks) {
        int8_t *base = lds + stage * C::STAGE_BYTES;
        const int k = ks * BK;
#pragma unroll
        for (int g = 0; g < C::WL; ++g)
            __builtin_amdgcn_global_load_lds((const void *)(wsrc[g] + k), (lds_ptr_t)(base + (C::WL * wave + g) * 1024), 16, 0, 0);
#pragma unroll
        for (int g = 0; g < C::XL; ++g)
            __builtin_amdgcn_global_load_lds((const void *)(xsrc[g] + k),
                                             (lds_ptr_t)(base + C::W_BYTES + (C::XL * wave + g) * 1024), 16, 0, 0);
    };

    // LDS side: lane reads row (lane%32) of a 32-row MFMA tile; for k quarter q
    // (32 k each) its 16 bytes are k chunk 2q + lane/32.
    const int frow = lane & 31;
    const int fsw = (frow >> 1) & 7;
    int foff[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) foff[q] = frow * BK + ((2 * q + (lane >> 5)) ^ fsw) * 16;
    auto read_frags = [&](int stage, v4i32 (&wf)[TN][4], v4i32 (&xf)[TM][4]) {
        const int8_t *wt = lds + stage * C::STAGE_BYTES + wn * 32 * TN * BK;
        const int8_t *xt = lds + stage * C::STAGE_BYTES + C::W_BYTES + wm * 32 * TM * BK;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
            for (int t = 0; t < TN; ++t) wf[t][q] = *reinterpret_cast<const v4i32 *>(wt + t * 32 * BK + foff[q]);
#pragma unroll
            for (int t = 0; t < TM; ++t) xf[t][q] = *reinterpret_cast<const v4i32 *>(xt + t * 32 * BK + foff[q]);
        }
    };

    v16i32 acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    auto mma = [&](const v4i32 (&wf)[TN][4], const v4i32 (&xf)[TM][4]) {
#pragma unroll
        for (int h = 0; h < 4; ++h)
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i][h], xf[j][h], acc[i][j], 0, 0, 0);
    };

    // One pipeline step.  The fragments of step ks are in registers.  Stage
    // (ks+1)%NST must have landed: of the loads this wavefront issued after it,
    // NST-2 stages' worth may still be in flight while new loads are being issued
    // (ISSUE), none after that.  After the barrier every wavefront has emptied
    // stage ks%NST into registers, so it takes the loads of step ks+NST.  The
    // fragments of step ks+1 are read while the MFMAs of step ks run: the step is
    // one basic block and the group barriers below spell out the interleaving
    // (MFMA first: the compiler's own wait for the current fragments must not
    // cover the new LDS reads).  Past the last step the read fetches a stale stage
    // that nobody uses.
    auto step = [&](auto issue_tag, int ks, const v4i32 (&cw)[TN][4], const v4i32 (&cx)[TM][4],
                    v4i32 (&nw)[TN][4], v4i32 (&nx)[TM][4]) {
        constexpr bool ISSUE = decltype(issue_tag)::value;
        if constexpr (ISSUE) wait_vmcnt<(NST - 2) * C::LPW>();
        else wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if constexpr (ISSUE) issue(ks % NST, ks + NST);
        read_frags((ks + 1) % NST, nw, nx);
        mma(cw, cx);
        // The global -> LDS loads come first in program order (the compiler keeps LDS
        // writes and LDS reads in order), two per MFMA; the fragment reads follow,
        // spread over the remaining MFMAs but the last.
        constexpr int N_MMA = 4 * TN * TM, N_DS = 4 * (TN + TM), N_VM = ISSUE ? C::LPW : 0;
        constexpr int VM_SLOTS = (N_VM + 1) / 2;
        constexpr int DS_PER = (N_DS + (N_MMA - VM_SLOTS - 1) - 1) / (N_MMA - VM_SLOTS - 1);
#pragma unroll
        for (int i = 0; i < N_MMA; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                         // one MFMA
            if (i < VM_SLOTS) __builtin_amdgcn_sched_group_barrier(0x010, 2, 0);       // global -> LDS loads
            else if ((i - VM_SLOTS) * DS_PER < N_DS)
                __builtin_amdgcn_sched_group_barrier(0x100, DS_PER, 0);                // LDS reads
        }
    };
    using issue_t = std::integral_constant<bool, true>;
    using drain_t = std::integral_constant<bool, false>;

    for (int s = 0; s < NST; ++s)
        if (s < ksteps) issue(s, s);
    if (ksteps >= NST) wait_vmcnt<(NST - 1) * C::LPW>();
    else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    v4i32 w0[TN][4], x0[TM][4], w1[TN][4], x1[TM][4];
    read_frags(0, w0, x0);
    const int n_issue = ksteps > NST ? ksteps - NST : 0;  // steps that still request a stage
    int ks = 0;
    for (; ks + 1 < n_issue; ks += 2) {
        step(issue_t{}, ks, w0, x0, w1, x1);
        step(issue_t{}, ks + 1, w1, x1, w0, x0);
    }
    if (ks < n_issue) {
        step(issue_t{}, ks, w0, x0, w1, x1);
        step(drain_t{}, ks + 1, w1, x1, w0, x0);
        ks += 2;
    }
    for (; ks + 1 < ksteps; ks += 2) {
        step(drain_t{}, ks, w0, x0, w1, x1);
        step(drain_t{}, ks + 1, w1, x1, w0, x0);
    }
    if (ks < ksteps) step(drain_t{}, ks, w0, x0, w1, x1);

    if constexpr (SPLIT) {
        // Accumulator element e of thread t at int e * THREADS + t of the workgroup's partial tile:
        // every instruction moves 256 contiguous bytes per wavefront.  The partials cross XCDs,
        // whose L2s are not coherent with each other: they are written and read as relaxed
        // device-scope atomics (stores that write through, loads that go to the coherence
        // point), ordered by "all my stores acknowledged" (vmcnt 0) before the arrival.  A device-
        // scope fence would do the same by writing back and invalidating the whole L2 under the
        // other workgroups' operand streams (measured: +25 us per launch).
        // What this relies on, all of it properties of gfx950 and not of the HIP memory model:
        //   - a relaxed agent-scope atomic store is emitted as global_store_dword ... sc1, which
        //     writes through the issuing XCD's L2 to memory (the point all XCDs agree on);
        //   - stores are counted by vmcnt on this ISA (gfx9 has no separate store counter), and a
        //     write-through store is acknowledged only once it has reached that point, so
        //     "s_waitcnt vmcnt(0)" below means every partial of this wavefront is visible chip-wide;
        //   - __syncthreads() then orders all wavefronts' acknowledged stores before thread 0's
        //     arrival atomic (a device-scope RMW executed at the same coherence point);
        //   - a relaxed agent-scope atomic load is global_load_dword ... sc1, which misses the local
        //     L2 and reads that point, so the last arriver cannot see a stale line.
        // A compiler that lowered these atomics differently, or a part whose vmcnt did not cover
        // write-through acknowledgement, would break this; test_linear_w8a8_bf16_split_k_same_bits
        // and the repeated-launch comparison against the unsplit kernel are the guard.
        constexpr int ELEMS = TN * TM * 16;
        int *mine = a.partials + ((size_t)split * tiles + tile) * (ELEMS * THREADS) + threadIdx.x;
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    __hip_atomic_store(mine + ((i * TM + j) * 16 + v) * THREADS, acc[i][j][v], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0)
            arrived_before = __hip_atomic_fetch_add(a.arrivals + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (arrived_before != a.splits - 1) return;  // uniform: not the last workgroup of the tile
        // all the others' elements are requested before the first is added (one trip to memory,
        // not one per split): four (two) splits' worth at a time, slots past the last split or on this
        // workgroup's own partial re-read split 0 and count for nothing
        constexpr int AT_A_TIME = ELEMS <= 32 ? 4 : 2;  // registers: 4 x 32 or 2 x 64 partial elements
        for (int s0 = 0; s0 < a.splits; s0 += AT_A_TIME) {
            int theirs[AT_A_TIME][ELEMS];
#pragma unroll
            for (int d = 0; d < AT_A_TIME; ++d) {
                const int s = s0 + d < a.splits ? s0 + d : 0;
                const int *src = a.partials + ((size_t)s * tiles + tile) * (ELEMS * THREADS) + threadIdx.x;
#pragma unroll
                for (int e = 0; e < ELEMS; ++e)
                    theirs[d][e] = __hip_atomic_load(src + e * THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int d = 0; d < AT_A_TIME; ++d) {
                const bool counts = s0 + d < a.splits && s0 + d != split;
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int j = 0; j < TM; ++j)
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc[i][j][v] += counts ? theirs[d][(i * TM + j) * 16 + v] : 0;
            }
        }
    }
    epilogue<TN, TM>(a, acc, lds, wave, lane, n0 + wn * 32 * TN, m0 + wm * 32 * TM, scales + wn * 32 * TN,
                     scales + C::BN + wm * 32 * TM);
}

template <int TN, int TM, int NST>
int launch(Args &a, hipStream_t st) {
    using C = Cfg<TN, TM, NST>;
    a.tiles_m = (a.M + C::BM - 1) / C::BM;
    a.tiles_n = (a.N + C::BN - 1) / C::BN;
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemm_w8a8_pipe_kernel<TN, TM, NST>),
                                   C::LDS_BYTES, devices, "cmi_gemm_w8a8"))
        return rc;
    a.warm_blocks = warm_workgroups(a.wq, (size_t)a.N * a.K, a.tiles_m * a.tiles_n);
    gemm_w8a8_pipe_kernel<TN, TM, NST><<<dim3(a.tiles_m * a.tiles_n + a.warm_blocks), dim3(THREADS), C::LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemm_w8a8");
}

// Split-K launch of the 64 x 64, the 128(m) x 64(n) or the 128 x 128 tile: a.splits, a.partials and
// a.arrivals set by the caller.
template <int TN, int TM, int NST>
int launch_split(Args &a, hipStream_t st) {
    using C = Cfg<TN, TM, NST>;
    a.tiles_m = (a.M + C::BM - 1) / C::BM;
    a.tiles_n = (a.N + C::BN - 1) / C::BN;
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemm_w8a8_pipe_kernel<TN, TM, NST, true>),
                                   C::LDS_BYTES, devices, "cmi_gemm_w8a8"))
        return rc;
    a.warm_blocks = warm_workgroups(a.wq, (size_t)a.N * a.K, a.tiles_m * a.tiles_n * a.splits);
    gemm_w8a8_pipe_kernel<TN, TM, NST, true><<<dim3(a.tiles_m * a.tiles_n * a.splits + a.warm_blocks), dim3(THREADS), C::LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemm_w8a8");
}

// ---------------------------------------------------------------------------
// 256 x 256 block tile, 8 wavefronts (2 along n x 4 along m, two per SIMD), each
// 128(n) x 64(m) = 4 x 2 MFMA tiles.  The operand bytes a CU must pull from L2
// per MFMA cycle halve against the 128 x 128 tile, which is what bounds that
// kernel.  LDS is a ring of five 32 KiB slots; the ring units alternate W tile,
// X tile of successive k steps (unit 2s = W of step s, unit 2s+1 = X of step s),
// so that beside the two units being computed from, up to three are in flight or
// landed -- with whole two-operand stages only two would fit and the memory
// pipe would drain at every step.  Fragments are double-buffered per k quarter
// (32 k), not per step, to stay within 256 registers.  One barrier per step:
// when the last quarter's fragments have been read the step's two slots are
// free and take units 2s+5, 2s+6, while units 2s+2, 2s+3 must have landed (only
// unit 2s+4 may still be in flight); those loads and the first fragments of
// step s+1 are issued under the last quarter's MFMAs.
namespace big {
constexpr int BM = 256, BN = 256, TN = 4, TM = 2;
constexpr int SLOT_BYTES = 256 * BK, SLOTS = 5;
constexpr int PARK_BYTES = 8 * 32 * TM * (64 * TN + 16);
constexpr int LDS_BYTES = SLOTS * SLOT_BYTES > PARK_BYTES ? SLOTS * SLOT_BYTES : PARK_BYTES;
constexpr int LPU = 4;  // loads per wavefront and unit
}  // namespace big

__global__ void __launch_bounds__(512, 2)
gemm_w8a8_big_kernel(const Args a) {
    using namespace big;
    extern __shared__ __align__(16) int8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave & 1, wm = wave >> 1;

    int tm, tn;
    tile_coords(a, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // Wavefront w fills rows 32w .. 32w+31 of an operand tile: 4 loads of
    // 8 rows x 128 B each; slot and swizzle as in the 4-wavefront kernel.
    const int lrow = lane >> 3;
    const int8_t *wsrc[4], *xsrc[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int row = (4 * wave + g) * 8 + lrow;
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        wsrc[g] = a.wq + (size_t)min(n0 + row, a.N - 1) * a.K + kc * 16;
        xsrc[g] = a.xq + (size_t)min(m0 + row, a.M - 1) * a.K + kc * 16;
    }
    // ring slot of a unit, as a byte offset
    auto slot_of = [](int unit) { return (unit % SLOTS) * SLOT_BYTES; };
    auto issue_w = [&](int ks) {
        int8_t *base = lds + slot_of(2 * ks) + (4 * wave) * 1024;
#pragma unroll
        for (int g = 0; g < 4; ++g)
            __builtin_amdgcn_global_load_lds((const void *)(wsrc[g] + ks * BK), (lds_ptr_t)(base + g * 1024), 16, 0, 0);
    };
    auto issue_x = [&](int ks) {
        int8_t *base = lds + slot_of(2 * ks + 1) + (4 * wave) * 1024;
#pragma unroll
        for (int g = 0; g < 4; ++g)
            __builtin_amdgcn_global_load_lds((const void *)(xsrc[g] + ks * BK), (lds_ptr_t)(base + g * 1024), 16, 0, 0);
    };

    const int frow = lane & 31;
    const int fsw = (frow >> 1) & 7;
    int foff[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) foff[q] = frow * BK + ((2 * q + (lane >> 5)) ^ fsw) * 16;
    struct Frag {
        v4i32 w[TN], x[TM];
    };
    auto read_q = [&](int ks, int q, Frag &f) {
        const int8_t *wt = lds + slot_of(2 * ks) + wn * 32 * TN * BK + foff[q];
        const int8_t *xt = lds + slot_of(2 * ks + 1) + wm * 32 * TM * BK + foff[q];
#pragma unroll
        for (int t = 0; t < TN; ++t) f.w[t] = *reinterpret_cast<const v4i32 *>(wt + t * 32 * BK);
#pragma unroll
        for (int t = 0; t < TM; ++t) f.x[t] = *reinterpret_cast<const v4i32 *>(xt + t * 32 * BK);
    };

    v16i32 acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    auto mma_q = [&](const Frag &f) {
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w[i], f.x[j], acc[i][j], 0, 0, 0);
    };
    // 8 MFMAs with the 6 fragment reads of the next quarter spread between them
    auto pace_quarter = [&]() {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };

    const int ksteps = a.K / BK;
    Frag f0, f1;
    // Step ks computes from units 2ks, 2ks+1 (first-quarter fragments in f0).
    // PHASE 2: steady state, two more units are requested (W of step ks+3 goes to
    // the slot of this step's X... no slot arithmetic is needed: unit u always
    // lives in slot u % 5, and units 2ks+5, 2ks+6 map onto the slots of 2ks, 2ks+1).
    // PHASE 1: only unit 2ks+5 exists (X of step ks+2).  PHASE 0: nothing left.
    auto step = [&](auto phase_tag, int ks) {
        constexpr int PHASE = decltype(phase_tag)::value;
        read_q(ks, 1, f1);
        mma_q(f0);
        pace_quarter();
        read_q(ks, 2, f0);
        mma_q(f1);
        pace_quarter();
        read_q(ks, 3, f1);
        mma_q(f0);
        pace_quarter();
        // this wavefront's reads of the step's slots are done; units 2ks+2, 2ks+3 landed
        if constexpr (PHASE == 2) wait_vmcnt<LPU>();
        else wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if constexpr (PHASE >= 1) issue_x(ks + 2);
        if constexpr (PHASE == 2) issue_w(ks + 3);
        read_q(ks + 1, 0, f0);  // past the last step: a stale slot nobody uses
        mma_q(f1);
        constexpr int VM_SLOTS = PHASE * 2;  // two loads per MFMA
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < VM_SLOTS) __builtin_amdgcn_sched_group_barrier(0x010, 2, 0);
            else if (i - VM_SLOTS < 3) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
    };
    using steady_t = std::integral_constant<int, 2>;
    using last_x_t = std::integral_constant<int, 1>;
    using drain_t = std::integral_constant<int, 0>;

    // Prologue: units 0..4 = W0 X0 W1 X1 W2.
    issue_w(0);
    issue_x(0);
    if (ksteps > 1) {
        issue_w(1);
        issue_x(1);
    }
    if (ksteps > 2) {
        issue_w(2);
        wait_vmcnt<3 * LPU>();
    } else if (ksteps > 1) {
        wait_vmcnt<2 * LPU>();
    } else {
        wait_vmcnt<0>();
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_q(0, 0, f0);
    // Step ks requests X of step ks+2 and W of step ks+3.
    int ks = 0;
    for (; ks + 3 < ksteps; ++ks) step(steady_t{}, ks);
    if (ks + 2 < ksteps) step(last_x_t{}, ks++);
    for (; ks < ksteps; ++ks) step(drain_t{}, ks);

    epilogue<TN, TM>(a, acc, lds, wave, lane, n0 + wn * 32 * TN, m0 + wm * 32 * TM);
}

int launch_big(Args &a, hipStream_t st) {
    a.tiles_m = (a.M + big::BM - 1) / big::BM;
    a.tiles_n = (a.N + big::BN - 1) / big::BN;
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemm_w8a8_big_kernel),
                                   big::LDS_BYTES, devices, "cmi_gemm_w8a8"))
        return rc;
    gemm_w8a8_big_kernel<<<dim3(a.tiles_m * a.tiles_n), dim3(512), big::LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemm_w8a8");
}

// ---------------------------------------------------------------------------
// 256(m) x 320(n) block tile, 8 wavefronts (2 along n x 4 along m, two per SIMD) of
// 64(m) x 160(n) = 2 x 5 MFMA tiles, 160 accumulator registers per lane.  Exists
// for the tile count: N = 9728 (Qwen3.5-4B's MLP width) is 38 x 256 but 30.4 x 320, so
// 2048 x 9728 is 248 of these tiles -- one round of the 256 CUs -- instead of 304 tiles of
// 256 x 256 (1.19 rounds).  It also needs the fewest L2 -> LDS bytes per MFMA of the three
// kernels.  Two LDS stages of 72 KiB, fragments double-buffered per k quarter, one barrier
// per step (structure of the 256 x 256 kernel without the slot ring).
namespace wide {
constexpr int BM = 256, BN = 320, TN = 5, TM = 2;
constexpr int W_BYTES = BN * BK, X_BYTES = BM * BK, STAGE_BYTES = W_BYTES + X_BYTES;
constexpr int PARK_BYTES = 8 * 32 * (64 * TN + 16);  // one m tile per epilogue pass
constexpr int OPERAND_BYTES = 2 * STAGE_BYTES > PARK_BYTES ? 2 * STAGE_BYTES : PARK_BYTES;
constexpr int LDS_BYTES = OPERAND_BYTES + 4 * (BN + BM);  // the tile's scales behind the stages
constexpr int WL = 5, XL = 4;  // loads per wavefront and stage
}  // namespace wide

__global__ void __launch_bounds__(512, 2)
gemm_w8a8_wide_kernel(const Args a) {
    using namespace wide;
    extern __shared__ __align__(16) int8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave & 1, wm = wave >> 1;

    int tm, tn;
    tile_coords(a, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    float *scales = reinterpret_cast<float *>(lds + OPERAND_BYTES);
    stage_scales<BN, BM>(a, scales, n0, m0);

    // Wavefront w fills W rows 40w .. 40w+39 and X rows 32w .. 32w+31 (8 rows x 128 B per load).
    // Addresses are a uniform base (tile corner, advanced by the k step) plus a 32-bit lane
    // offset: 9 registers instead of 18 for 64-bit pointers, which this kernel cannot spare.
    const int lrow = lane >> 3;
    uint32_t woff[WL], xoff[XL];
#pragma unroll
    for (int g = 0; g < WL; ++g) {
        const int row = (WL * wave + g) * 8 + lrow;
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        woff[g] = (uint32_t)min(row, a.N - 1 - n0) * (uint32_t)a.K + kc * 16;
    }
#pragma unroll
    for (int g = 0; g < XL; ++g) {
        const int row = (XL * wave + g) * 8 + lrow;
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        xoff[g] = (uint32_t)min(row, a.M - 1 - m0) * (uint32_t)a.K + kc * 16;
    }
    const int8_t *wtile = a.wq + (size_t)n0 * a.K, *xtile = a.xq + (size_t)m0 * a.K;
    auto issue = [&](int stage, int ks) {
        int8_t *base = lds + stage * STAGE_BYTES;
        const int8_t *wk = wtile + ks * BK, *xk = xtile + ks * BK;
#pragma unroll
        for (int g = 0; g < WL; ++g)
            __builtin_amdgcn_global_load_lds((const void *)(wk + woff[g]),
                                             (lds_ptr_t)(base + (WL * wave + g) * 1024), 16, 0, 0);
#pragma unroll
        for (int g = 0; g < XL; ++g)
            __builtin_amdgcn_global_load_lds((const void *)(xk + xoff[g]),
                                             (lds_ptr_t)(base + W_BYTES + (XL * wave + g) * 1024), 16, 0, 0);
    };

    const int frow = lane & 31;
    const int fsw = (frow >> 1) & 7;
    int foff[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) foff[q] = frow * BK + ((2 * q + (lane >> 5)) ^ fsw) * 16;
    struct Frag {
        v4i32 w[TN], x[TM];
    };
    auto read_q = [&](int stage, int q, Frag &f) {
        const int8_t *wt = lds + stage * STAGE_BYTES + wn * 32 * TN * BK + foff[q];
        const int8_t *xt = lds + stage * STAGE_BYTES + W_BYTES + wm * 32 * TM * BK + foff[q];
#pragma unroll
        for (int t = 0; t < TN; ++t) f.w[t] = *reinterpret_cast<const v4i32 *>(wt + t * 32 * BK);
#pragma unroll
        for (int t = 0; t < TM; ++t) f.x[t] = *reinterpret_cast<const v4i32 *>(xt + t * 32 * BK);
    };

    v16i32 acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    auto mma_q = [&](const Frag &f) {
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w[i], f.x[j], acc[i][j], 0, 0, 0);
    };
    constexpr int N_MMA = TN * TM, N_DS = TN + TM;
    // a quarter's MFMAs with the fragment reads of the next quarter spread between them
    auto pace_quarter = [&]() {
#pragma unroll
        for (int i = 0; i < N_MMA; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < N_DS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };

    const int ksteps = a.K / BK;
    Frag f0, f1;
    // Step ks computes from stage ks%2 (first-quarter fragments in f0).  When the last
    // quarter's fragments have been read the stage is free for step ks+2, and the other
    // stage (requested a step ago) must have landed.
    auto step = [&](auto issue_tag, int ks) {
        constexpr bool ISSUE = decltype(issue_tag)::value;
        const int cur = ks & 1;
        read_q(cur, 1, f1);
        mma_q(f0);
        pace_quarter();
        read_q(cur, 2, f0);
        mma_q(f1);
        pace_quarter();
        read_q(cur, 3, f1);
        mma_q(f0);
        pace_quarter();
        wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if constexpr (ISSUE) issue(cur, ks + 2);
        read_q(cur ^ 1, 0, f0);  // past the last step: a stale stage nobody uses
        mma_q(f1);
        constexpr int N_VM = ISSUE ? WL + XL : 0;
#pragma unroll
        for (int i = 0; i < N_MMA; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (2 * i < N_VM) __builtin_amdgcn_sched_group_barrier(0x010, 2, 0);
            else if (i - (N_VM + 1) / 2 < N_DS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };
    using issue_t = std::integral_constant<bool, true>;
    using drain_t = std::integral_constant<bool, false>;

    issue(0, 0);
    if (ksteps > 1) {
        issue(1, 1);
        wait_vmcnt<9>();
    } else {
        wait_vmcnt<0>();
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_q(0, 0, f0);
    int ks = 0;
    for (; ks + 2 < ksteps; ++ks) step(issue_t{}, ks);
    for (; ks < ksteps; ++ks) step(drain_t{}, ks);

    epilogue<TN, TM, 1>(a, acc, lds, wave, lane, n0 + wn * 32 * TN, m0 + wm * 32 * TM, scales + wn * 32 * TN,
                        scales + BN + wm * 32 * TM);
}

int launch_wide(Args &a, hipStream_t st) {
    a.tiles_m = (a.M + wide::BM - 1) / wide::BM;
    a.tiles_n = (a.N + wide::BN - 1) / wide::BN;
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemm_w8a8_wide_kernel),
                                   wide::LDS_BYTES, devices, "cmi_gemm_w8a8"))
        return rc;
    gemm_w8a8_wide_kernel<<<dim3(a.tiles_m * a.tiles_n), dim3(512), wide::LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemm_w8a8");
}

// ---------------------------------------------------------------------------
// The same 256(m) x 320(n) tile walked weight tile by weight tile inside a K step, so that a
// stage is handed back in pieces and its next contents are in flight for about a step and a half
// instead of one step.  The two-stage kernel above reads every row of a stage in each of the
// four k quarters, so nothing of a stage is free before the step's last quarter and a stage's 72 KiB
// are requested one step (about 1.2 us of MFMAs) before they are needed.  Here a wavefront keeps the
// step's activation fragments in registers (8 x 16 bytes, all four quarters) and goes through its
// five 32-row weight tiles one after the other, in ten "half groups" of 4 MFMAs (weight tile I,
// k quarters 2H and 2H+1, against both activation tiles): the activation rows of a stage and weight
// tiles 0, 1 are free three tenths into the step, tiles 2..4 nine tenths.  Two barriers per step
// (A in half group 3, B in half group 9) hand the freed rows to the requests of step ks+2:
//     A(ks): X(ks+2), W tiles 0, 1 (ks+2)      B(ks): W tiles 2..4 (ks+2)
// and certify what the next reads need: at B(ks) every wavefront's share of X(ks+1) and W 0, 1
// (ks+1) has landed (requested at A(ks-1)), at A(ks) W 2..4 (ks) (requested at B(ks-2)); a
// wavefront requests 6 + 3 loads per step, so both waits are vmcnt(9).
//
// Fragment reads are issued where the compiler does not see them (inline ds_read_b128) and
// waited for with exact counts: left to itself the compiler drains the LDS queue (lgkmcnt(0)) in
// front of every use, so a read never has more than the few MFMAs between it and its use to
// land -- measured 12 us of a 50 us launch.  Here the fragments of half group k+2 are read during
// half group k into one of three fragment buffers (LDS returns in order, so the wait in front of
// half group k is "all but the reads issued since": lgkmcnt(2)), except where the data is
// certified only at a barrier (half groups 4 and 5 are read together behind A, 0 and 1 of the next
// step behind B).  Which buffer a half group uses is a fixed table per step parity, chosen so that
// a read never lands in a buffer that a pending half group still needs.
// Requests are buffer loads (buffer_load_dwordx4 ... lds): one 32-bit lane offset per operand, the
// tile / step / row-group offset in a scalar register, rows past the matrix read as zeros.
// Same MFMAs on the same operands per accumulator, in the same k order: the accumulators, and so
// the bits, are those of the two-stage kernel.
namespace tilewise {
// fragment buffer of half group k in a step of parity P
constexpr int BUF[2][10] = {{0, 2, 1, 0, 2, 1, 0, 2, 1, 0}, {1, 2, 0, 1, 2, 0, 1, 2, 0, 1}};
__device__ __forceinline__ uint32_t lds_offset(const void *p) { return (uint32_t)(uintptr_t)(lds_ptr_t)p; }
template <int IMM>
__device__ __forceinline__ void read16(v4i32 &d, uint32_t base) {
    static_assert(IMM >= 0 && IMM < 65536, "LDS immediate offset");
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(d) : "v"(base), "n"(IMM) : "memory");
}
// the registers named are not used before the LDS queue is down to N reads
template <int N>
__device__ __forceinline__ void lds_wait(v4i32 &f0, v4i32 &f1) {
    if constexpr (N == 0) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f0), "+v"(f1)::"memory");
    else if constexpr (N == 2) asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(f0), "+v"(f1)::"memory");
    else static_assert(N < 0, "add the lgkmcnt literal");
}
template <int N>
__device__ __forceinline__ void lds_wait(v4i32 &f0, v4i32 &f1, v4i32 &x0, v4i32 &x1, v4i32 &x2, v4i32 &x3) {
    if constexpr (N == 2)
        asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(f0), "+v"(f1), "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3)::"memory");
    else if constexpr (N == 6)
        asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(f0), "+v"(f1), "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3)::"memory");
    else static_assert(N < 0, "add the lgkmcnt literal");
}
template <int IMM>
__device__ __forceinline__ void read4(uint32_t &d, uint32_t base) {
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(d) : "v"(base), "n"(IMM) : "memory");
}
// A step of the persistent kernel next to a tile boundary differs from the plain one: the first
// step of a tile starts its accumulators from zero, requests the tile's scales and, like the A
// barrier of the second, has nothing to wait for in memory (the epilogue, or the prologue, before it
// ended with every request landed); the last step of a tile leaves the next step's fragment reads
// to whoever comes after the epilogue, which needs the registers.
enum { STEP_PLAIN = 0, STEP_FIRST = 1, STEP_SECOND = 2, STEP_LAST = 3 };
constexpr int SCALE_SLOTS = 16;  // persistent kernel: 256-byte pieces of the scale area, one per request
}  // namespace tilewise

// Epilogue of the persistent kernel for one wavefront tile of 5 x 2 MFMA tiles (corner: column
// n0 + 160 (wave & 1), row m0 + 64 (wave / 2) of the matrix): scale, narrow, and write from
// registers, touching no operand stage.  A lane holds, per MFMA tile and q, 4 consecutive columns of
// its row (8 bytes of bf16); v_permlane32_swap trades one of each pair of such pieces with the lane
// 32 up, which holds the columns in between, so that each lane owns 8 consecutive columns per
// store: 20 stores of 16 bytes per wavefront.  They are buffer stores -- rows past M fall outside
// the resource and are dropped, columns past N get an offset that does; N % 8 == 0 -- so every
// wavefront issues all 20 whatever the tile.  The scales come from LDS at `scales_lds` (320 column
// scales, then 256 row scales) through reads the compiler does not see: it would otherwise wait
// for every request in flight, which are LDS writes to it.  Before the first store every request of
// the wavefront has landed (vmcnt(0): by then the loads for the next tile's first two steps are
// some microseconds old), so the vmcnt waits of the steps that follow never depend on how stores
// and loads are retired relative to each other.
__device__ __forceinline__ void epilogue_direct(const Args &a, v16i32 (&acc)[5][2], __amdgpu_buffer_rsrc_t yres,
                                                uint32_t scales_lds, int wave, int n0, int m0) {
    using namespace tilewise;
    // the lane number anew, where the compiler cannot move it (and what is derived from it) out of
    // the tile loop: the K steps have no registers to spare for the epilogue's addresses
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=&v"(lane));
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef unsigned u32x2_swap __attribute__((ext_vector_type(2)));
    const int wn = wave & 1, wm = wave >> 1, h = lane >> 5, r = lane & 31;
    const uint32_t ws_base = scales_lds + (wn * 160 + 4 * h) * 4;
    const uint32_t xs_base = scales_lds + (wide::BN + wm * 64 + r) * 4;
    uint32_t xm_bits[2];
    read4<0>(xm_bits[0], xs_base);
    read4<128>(xm_bits[1], xs_base);
    u32x4 out[5][2][2];
    using std::integral_constant;
    auto tile_row = [&](auto i_tag) {
        constexpr int I = decltype(i_tag)::value;
        v4i32 wsv[4];
        read16<(32 * I + 0) * 4>(wsv[0], ws_base);
        read16<(32 * I + 8) * 4>(wsv[1], ws_base);
        read16<(32 * I + 16) * 4>(wsv[2], ws_base);
        read16<(32 * I + 24) * 4>(wsv[3], ws_base);
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(wsv[0]), "+v"(wsv[1]), "+v"(wsv[2]), "+v"(wsv[3]), "+v"(xm_bits[0]), "+v"(xm_bits[1])::"memory");
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const float xm = __uint_as_float(xm_bits[j]);
            uint32_t d[4][2];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float t[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) t[e] = ((float)acc[I][j][4 * q + e] * xm) * __int_as_float(wsv[q][e]);
                d[q][0] = pack_bf16(t[0], t[1]);
                d[q][1] = pack_bf16(t[2], t[3]);
            }
            // pieces 2p and 2p+1 hold columns 16p + 4h .. and 16p + 8 + 4h ..: the lower lane hands
            // its 2p+1 up and gets the upper lane's 2p, after which lane half h owns 16p + 8h .. + 7
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const u32x2_swap s0 = __builtin_amdgcn_permlane32_swap(d[2 * p][0], d[2 * p + 1][0], false, false);
                const u32x2_swap s1 = __builtin_amdgcn_permlane32_swap(d[2 * p][1], d[2 * p + 1][1], false, false);
                out[I][j][p] = u32x4{s0.x, s1.x, s0.y, s1.y};
            }
        }
    };
    tile_row(integral_constant<int, 0>{});
    tile_row(integral_constant<int, 1>{});
    tile_row(integral_constant<int, 2>{});
    tile_row(integral_constant<int, 3>{});
    tile_row(integral_constant<int, 4>{});
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    const int ncols = a.N - (n0 + wn * 160 + 8 * h);  // columns left from this lane's first
    const uint32_t ytile = (uint32_t)(((size_t)m0 * a.ldy + n0) * 2);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t voff = (uint32_t)(((wm * 64 + 32 * j + r) * a.ldy + wn * 160 + 8 * h) * 2);
#pragma unroll
        for (int i = 0; i < 5; ++i)
#pragma unroll
            for (int p = 0; p < 2; ++p)
                __builtin_amdgcn_raw_buffer_store_b128(out[i][j][p], yres,
                                                       32 * i + 16 * p < ncols ? voff + (32 * i + 16 * p) * 2 : 0x80000000u,
                                                       ytile, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
}

template <bool PERSIST>
__global__ void __launch_bounds__(512, 2)
gemm_w8a8_wide_tilewise_kernel(const Args a) {
    using namespace wide;
    using namespace tilewise;
    extern __shared__ __align__(16) int8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave & 1, wm = wave >> 1;

    const int tiles = a.tiles_m * a.tiles_n;
    int tm, tn;
    tile_coords(a, tm, tn);
    int m0 = tm * BM, n0 = tn * BN;
    float *scales = reinterpret_cast<float *>(lds + OPERAND_BYTES);
    if constexpr (!PERSIST) stage_scales<BN, BM>(a, scales, n0, m0);

    // LDS: weights as [n half][stage][160 rows], activations behind them as [m quarter][stage][64 rows],
    // so that both stages of a wavefront's rows are within the 64 KiB reach of an LDS instruction's
    // immediate offset and one base register per k quarter serves a whole operand.
    constexpr int W_HALF = 160 * BK, X_QUARTER = 64 * BK, X_BASE = 4 * W_HALF;
    // Requests.  Weight tile i of n half h is rows 160 h + 32 i .. + 31; its 64 rows (both halves)
    // are 8 loads of 8 rows, one per wavefront: wavefront w takes rows 160 (w & 1) + 32 i + 8 (w >> 1)
    // .. + 7.  X rows 32 w + 8 g .. + 7, g = 0..3.  Lane i of a load lands in slot i of the 1 KiB:
    // row i / 8, stored chunk i % 8, which holds k chunk (i % 8) ^ ((row / 2) % 8).
    // A buffer access is checked against the resource's size with the scalar offset included
    // (measured on gfx950: lane offset 0 + scalar offset past the end reads 0), so the tile corner
    // can live in the scalar offset and rows past the matrix still read as zeros.
    const int lrow = lane >> 3;
    const int wrow = wn * 160 + wm * 8 + lrow;  // + 32 i: the swizzle does not depend on i
    const uint32_t wvoff = (uint32_t)wrow * (uint32_t)a.K + (((lane & 7) ^ ((wrow >> 1) & 7)) * 16);
    const int xrow = XL * wave * 8 + lrow;      // + 8 g: odd g flip bit 2 of the swizzle
    uint32_t xvoff[2];
#pragma unroll
    for (int g = 0; g < 2; ++g)
        xvoff[g] = (uint32_t)xrow * (uint32_t)a.K + (((lane & 7) ^ (((xrow + 8 * g) >> 1) & 7)) * 16);
    const __amdgpu_buffer_rsrc_t wres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(a.wq), 0, (int)((size_t)a.N * a.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t xres =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(a.xq), 0, (int)((size_t)a.M * a.K), 0x00020000);
    uint32_t wtile = (uint32_t)n0 * (uint32_t)a.K, xtile = (uint32_t)m0 * (uint32_t)a.K;
    const uint32_t k32 = 32u * (uint32_t)a.K, k8 = 8u * (uint32_t)a.K;
    int8_t *const wslot = lds + wn * 2 * W_HALF + wm * 8 * BK;                              // weight tile 0, stage 0
    int8_t *const xslot = lds + X_BASE + (wave >> 1) * 2 * X_QUARTER + (wave & 1) * 4 * 1024;  // g = 0, stage 0
    // step ks of the tile whose corner offsets are wt / xt
    auto issue_w = [&](int stage, uint32_t wt, int ks, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(wres, (lds_ptr_t)(wslot + stage * W_HALF + i * 32 * BK), 16, wvoff,
                                                 wt + i * k32 + ks * BK, 0, 0);
    };
    auto issue_a = [&](int stage, uint32_t wt, uint32_t xt, int ks) {
#pragma unroll
        for (int g = 0; g < XL; ++g)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(xres, (lds_ptr_t)(xslot + stage * X_QUARTER + g * 1024), 16,
                                                     xvoff[g & 1], xt + g * k8 + ks * BK, 0, 0);
        issue_w(stage, wt, ks, 0);
        issue_w(stage, wt, ks, 1);
    };
    auto issue_b = [&](int stage, uint32_t wt, int ks) {
        issue_w(stage, wt, ks, 2);
        issue_w(stage, wt, ks, 3);
        issue_w(stage, wt, ks, 4);
    };
    // Persistent kernel: the scales of the tile whose corner is (n_, m_), two requests of 64 floats
    // per wavefront (every wavefront issues the same number of loads: the vmcnt waits count them):
    // pieces 0..4 the 320 column scales, 5..8 the 256 row scales, the rest unused; past the matrix zeros.
    auto issue_scales = [&](int n_, int m_) {
        const __amdgpu_buffer_rsrc_t wsres =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.ws), 0, a.N * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t xsres =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.xs), 0, a.M * 4, 0x00020000);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int q = 2 * wave + e;
            const lds_ptr_t dst = (lds_ptr_t)(lds + OPERAND_BYTES + q * 256);
            if (q >= 5 && q < 9)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(xsres, dst, 4, lane * 4, (m_ + 64 * (q - 5)) * 4, 0, 0);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(wsres, dst, 4, lane * 4, (n_ + (q < 5 ? 64 * q : 0)) * 4, 0, 0);
        }
    };

    // Fragment reads: lane reads row (lane % 32) of a 32-row MFMA tile; for k quarter q its 16 bytes
    // are k chunk 2q + lane / 32 (swizzled).  One base per quarter and operand, the rest immediates.
    const int frow = lane & 31;
    const int fsw = (frow >> 1) & 7;
    uint32_t wbase[4], xbase[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int foff = frow * BK + ((2 * q + (lane >> 5)) ^ fsw) * 16;
        wbase[q] = lds_offset(lds + wn * 2 * W_HALF) + foff;
        xbase[q] = lds_offset(lds + X_BASE + wm * 2 * X_QUARTER) + foff;
    }
    v4i32 xf[TM][4];  // the step's activation fragments, all four k quarters
    v4i32 wf[3][2];   // two k quarters of one weight tile, three buffers
    using std::integral_constant;
#define IC(v) integral_constant<int, (v)>{}
    // fragments of half group K of a step of parity P (its operands are in stage P)
    auto read_w = [&](auto parity_tag, auto hg_tag) {
        constexpr int P = decltype(parity_tag)::value, K = decltype(hg_tag)::value, I = K / 2, H = K % 2;
        read16<P * W_HALF + I * 32 * BK>(wf[BUF[P][K]][0], wbase[2 * H]);
        read16<P * W_HALF + I * 32 * BK>(wf[BUF[P][K]][1], wbase[2 * H + 1]);
    };
    // activation quarters 2H, 2H+1 of a step of parity P
    auto read_x = [&](auto parity_tag, auto half_tag) {
        constexpr int P = decltype(parity_tag)::value, H = decltype(half_tag)::value;
#pragma unroll
        for (int q = 2 * H; q < 2 * H + 2; ++q) {
            read16<P * X_QUARTER>(xf[0][q], xbase[q]);
            read16<P * X_QUARTER + 32 * BK>(xf[1][q], xbase[q]);
        }
    };

    v16i32 acc[TN][TM];
    if constexpr (!PERSIST) {
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    }
    // the 4 MFMAs of half group K in a step of parity P; FRESH: the accumulators start from zero
    // (the first MFMA into each takes the constant as its addend)
    auto mma = [&](auto parity_tag, auto hg_tag, auto fresh_tag) {
        constexpr int P = decltype(parity_tag)::value, K = decltype(hg_tag)::value, I = K / 2, H = K % 2;
        constexpr bool FRESH = decltype(fresh_tag)::value != 0 && H == 0;
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                v16i32 c = acc[I][j];
                if (FRESH && q == 0)
#pragma unroll
                    for (int v = 0; v < 16; ++v) c[v] = 0;
                acc[I][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[BUF[P][K]][q], xf[j][2 * H + q], c, 0, 0, 0);
            }
    };
    // the wait in front of half group K: N reads were issued after its fragments
    auto wait_w = [&](auto parity_tag, auto hg_tag, auto n_tag) {
        constexpr int P = decltype(parity_tag)::value, K = decltype(hg_tag)::value, N = decltype(n_tag)::value;
        lds_wait<N>(wf[BUF[P][K]][0], wf[BUF[P][K]][1]);
    };
    auto wait_wx = [&](auto parity_tag, auto hg_tag, auto n_tag) {
        constexpr int P = decltype(parity_tag)::value, K = decltype(hg_tag)::value, N = decltype(n_tag)::value, H = K % 2;
        lds_wait<N>(wf[BUF[P][K]][0], wf[BUF[P][K]][1], xf[0][2 * H], xf[1][2 * H], xf[0][2 * H + 1], xf[1][2 * H + 1]);
    };
    auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
    // the first fragments of a tile's first step (half groups 0 and 1 of a step of parity 0)
    auto read_first = [&]() {
        read_w(IC(0), IC(0));
        read_x(IC(0), IC(0));
        read_w(IC(0), IC(1));
        read_x(IC(0), IC(1));
        fence();
    };

    const int ksteps = a.K / BK;
    // One K step from stage P.  On entry the fragments of half groups 0 and 1 are on their way (12
    // reads, issued in that order).  Its requests are step `rks` of the tile at rw / rx: two steps
    // ahead; past the end of the last tile the last step's operands once more instead of nothing
    // (into rows that are free, nobody reads them), so that every step issues the same 9 loads and
    // both vmcnt waits are 9 throughout.
    auto step = [&](auto p, auto kind_tag, uint32_t rw, uint32_t rx, int rks) {
        constexpr int P = decltype(p)::value, KIND = decltype(kind_tag)::value;
        constexpr auto np = IC(P ^ 1);
        constexpr auto fresh = IC(KIND == STEP_FIRST ? 1 : 0);
        wait_wx(p, IC(0), IC(6));
        mma(p, IC(0), fresh);
        read_w(p, IC(2));
        fence();
        wait_wx(p, IC(1), IC(2));
        mma(p, IC(1), fresh);
        read_w(p, IC(3));
        fence();
        wait_w(p, IC(2), IC(2));
        mma(p, IC(2), fresh);
        fence();
        // A: X and weight tiles 0, 1 of this stage are in registers everywhere; tiles 2..4 have landed
        wait_w(p, IC(3), IC(0));
        if constexpr (KIND != STEP_FIRST && KIND != STEP_SECOND) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue_a(P, rw, rx, rks);
        if constexpr (KIND == STEP_FIRST) issue_scales(n0, m0);
        read_w(p, IC(4));
        read_w(p, IC(5));
        mma(p, IC(3), fresh);
        fence();
        wait_w(p, IC(4), IC(2));
        mma(p, IC(4), fresh);
        read_w(p, IC(6));
        fence();
        wait_w(p, IC(5), IC(2));
        mma(p, IC(5), fresh);
        read_w(p, IC(7));
        fence();
        wait_w(p, IC(6), IC(2));
        mma(p, IC(6), fresh);
        read_w(p, IC(8));
        fence();
        wait_w(p, IC(7), IC(2));
        mma(p, IC(7), fresh);
        read_w(p, IC(9));
        fence();
        wait_w(p, IC(8), IC(2));
        mma(p, IC(8), fresh);
        fence();
        // B: weight tiles 2..4 are in registers everywhere; X and tiles 0, 1 of the next step have landed
        wait_w(p, IC(9), IC(0));
        if constexpr (KIND != STEP_FIRST) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue_b(P, rw, rks);
        if constexpr (KIND == STEP_LAST) {
            fence();
            mma(p, IC(9), fresh);
            fence();
        } else {
            // the next step's first fragments (past the last step: a stale stage, nobody uses them);
            // its quarters 2, 3 of X replace the ones this half group still multiplies, so they follow it
            read_w(np, IC(0));
            read_x(np, IC(0));
            fence();
            mma(p, IC(9), fresh);
            fence();
            read_w(np, IC(1));
            read_x(np, IC(1));
            fence();
        }
    };

    // Prologue: both stages requested in the order the steps request them (A then B).
    // The persistent kernel waits for all of it: its first tile then starts like every other, behind an
    // epilogue that left no request in flight.
    issue_a(0, wtile, xtile, 0);
    issue_b(0, wtile, 0);
    issue_a(1, wtile, xtile, min(1, ksteps - 1));
    issue_b(1, wtile, min(1, ksteps - 1));
    if constexpr (PERSIST) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_first();

    if constexpr (!PERSIST) {
        int ks = 0;
        for (; ks + 1 < ksteps; ks += 2) {
            step(IC(0), IC(STEP_PLAIN), wtile, xtile, min(ks + 2, ksteps - 1));
            step(IC(1), IC(STEP_PLAIN), wtile, xtile, min(ks + 3, ksteps - 1));
        }
        if (ks < ksteps) step(IC(0), IC(STEP_PLAIN), wtile, xtile, ksteps - 1);
        // the stale fragment reads and the repeated requests of the last steps must be over before their
        // registers and the stages are used for anything else
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        fence();
        epilogue<TN, TM, 1>(a, acc, lds, wave, lane, n0 + wn * 32 * TN, m0 + wm * 32 * TM, scales + wn * 32 * TN,
                            scales + BN + wm * 32 * TM);
    } else {
        // Tiles blockIdx.x, + gridDim.x, ...: an even number (>= 4) of K steps each, so that a tile
        // starts in stage 0.  The last two steps of a tile request the first two of the next, the
        // epilogue touches no operand stage (results go from registers to memory, scales from
        // their own corner of LDS), so the pipeline runs on across the boundary.
        const __amdgpu_buffer_rsrc_t yres = __builtin_amdgcn_make_buffer_rsrc(
            a.y, 0, (int)((((size_t)a.M - 1) * a.ldy + a.N) * 2), 0x00020000);
        int tile = blockIdx.x;
        while (true) {
            const int next = tile + gridDim.x;
            const bool more = next < tiles;
            int m1 = m0, n1 = n0;
            if (more) {
                tile_coords(a, tm, tn, next);
                m1 = tm * BM, n1 = tn * BN;
            }
            const uint32_t wnext = (uint32_t)n1 * (uint32_t)a.K, xnext = (uint32_t)m1 * (uint32_t)a.K;
            step(IC(0), IC(STEP_FIRST), wtile, xtile, 2);
            step(IC(1), IC(STEP_SECOND), wtile, xtile, 3);
            for (int ks = 2; ks < ksteps - 2; ks += 2) {
                step(IC(0), IC(STEP_PLAIN), wtile, xtile, ks + 2);
                step(IC(1), IC(STEP_PLAIN), wtile, xtile, ks + 3);
            }
            step(IC(0), IC(STEP_PLAIN), wnext, xnext, more ? 0 : ksteps - 1);
            step(IC(1), IC(STEP_LAST), wnext, xnext, more ? 1 : ksteps - 1);
            epilogue_direct(a, acc, yres, lds_offset(scales), wave, n0, m0);
            if (!more) break;
            tile = next, m0 = m1, n0 = n1, wtile = wnext, xtile = xnext;
            read_first();
        }
    }
#undef IC
}

int launch_wide(Args &a, hipStream_t st);

int launch_wide_tilewise(Args &a, hipStream_t st) {
    // buffer offsets are 32 bits: matrices (and the tile rows past their end) must stay below 2 GiB
    if ((size_t)(a.N + wide::BN) * a.K >= ((size_t)1 << 31) || (size_t)(a.M + wide::BM) * a.K >= ((size_t)1 << 31))
        return launch_wide(a, st);
    a.tiles_m = (a.M + wide::BM - 1) / wide::BM;
    a.tiles_n = (a.N + wide::BN - 1) / wide::BN;
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemm_w8a8_wide_tilewise_kernel<false>),
                                   wide::LDS_BYTES, devices, "cmi_gemm_w8a8"))
        return rc;
    gemm_w8a8_wide_tilewise_kernel<false><<<dim3(a.tiles_m * a.tiles_n), dim3(512), wide::LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemm_w8a8");
}

// The persistent form: one workgroup per CU walks tiles blockIdx.x, + grid, ...  Takes what the
// direct epilogue can write (bf16 rows of 16-byte pieces, no int32 dump) and an even number of K
// steps; anything else goes to the one-tile-per-workgroup kernel.
int launch_wide_persistent(Args &a, hipStream_t st) {
    const int ksteps = a.K / BK;
    const bool fits = !a.acc_out && a.N % 8 == 0 && a.ldy % 8 == 0 && aligned(a.y, 16) && ksteps >= 4 && ksteps % 2 == 0 &&
                      ((size_t)a.M + wide::BM) * a.ldy * 2 < ((size_t)1 << 31) &&
                      (size_t)(a.N + wide::BN) * a.K < ((size_t)1 << 31) && (size_t)(a.M + wide::BM) * a.K < ((size_t)1 << 31);
    if (!fits) return launch_wide_tilewise(a, st);
    a.tiles_m = (a.M + wide::BM - 1) / wide::BM;
    a.tiles_n = (a.N + wide::BN - 1) / wide::BN;
    constexpr int LDS = wide::OPERAND_BYTES + tilewise::SCALE_SLOTS * 256;
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemm_w8a8_wide_tilewise_kernel<true>), LDS, devices,
                                   "cmi_gemm_w8a8"))
        return rc;
    const int tiles = a.tiles_m * a.tiles_n, cus = compute_units();
    CMI_REQUIRE(cus > 0, CMI_E_HIP, "cmi_gemm_w8a8: cannot read the device's compute unit count");
    gemm_w8a8_wide_tilewise_kernel<true><<<dim3(tiles < cus ? tiles : cus), dim3(512), LDS, st>>>(a);
    return check_launch("cmi_gemm_w8a8");
}

}  // namespace

extern "C" int cmi_gemm_w8a8(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws,
                             void *y, int32_t *acc_out, int M, int N, int K, int ldy,
                             void *stream) {
    return cmi::gemm_w8a8_split(xq, wq, xs, ws, y, acc_out, M, N, K, ldy, nullptr, nullptr, 0, stream);
}

size_t cmi::gemm_w8a8_split_bytes(int M, int N, int K) {
    if (M <= 16 || K % BK != 0 || N < 8) return 0;
    // up to 256 workgroups of 64 x 64 or 128 x 64 int32 each, whatever the split
    if (M <= 256) return (size_t)256 * 128 * 64 * 4;
    // up to 1024 rows of a narrow, long projection (at most 128 tiles of 128 x 128, 16 K steps and
    // more): up to 256 workgroups of 128 x 128 int32
    const int tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
    return M <= 1024 && tiles128 <= 128 && K / BK >= 16 ? (size_t)256 * 128 * 128 * 4 : 0;
}

int cmi::gemm_w8a8_split(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws, void *y,
                         int32_t *acc_out, int M, int N, int K, int ldy, int *arrivals, void *partials,
                         size_t partial_bytes, void *stream) {
    CMI_REQUIRE(M >= 0 && N >= 1 && K >= 16, CMI_E_ARG, "cmi_gemm_w8a8: bad shape M=%d N=%d K=%d", M, N, K);
    if (M == 0) return CMI_OK;  // an empty batch has no storage to point at
    CMI_REQUIRE(xq && wq && xs && ws && y, CMI_E_ARG, "cmi_gemm_w8a8: null pointer");
    CMI_REQUIRE(ldy >= N, CMI_E_ARG, "cmi_gemm_w8a8: ldy=%d is smaller than N=%d", ldy, N);
    CMI_REQUIRE(K % 16 == 0, CMI_E_UNSUPPORTED, "cmi_gemm_w8a8: K=%d is not a multiple of 16", K);
    CMI_REQUIRE(aligned(xq, 16) && aligned(wq, 16), CMI_E_ARG,
                "cmi_gemm_w8a8: xq and wq must be 16-byte aligned");
    const int force = option_gemm_tile();
    if (M <= 16 && !force) {
        // a verify-sized batch: read the weight once, GEMV style
        const int rc = gemm_w8a8_rows16(xq, wq, xs, ws, y, acc_out, M, N, K, ldy, stream);
        if (rc != CMI_E_UNSUPPORTED) return rc;
    }
    int mid = 0;  // 17..256 rows: the tile kernel the cost models below chose (64 x 64: 6464), if any
    if (M > 16 && M <= 256 && K % BK == 0 && N >= 8 && !force) {
        // Between the GEMV-like batch and the full tile pipeline every kernel is bound by what its
        // workgroups pull through L2 per dependent step, and which one is fastest changes with the
        // shape: the read-once kernel pays per 16-row chunk, a tile kernel K / 128 steps whose
        // length grows with N (bytes per step) and with the rounds of workgroups on the 256 CUs.
        // Cost models (us) fitted to cold-weight measurements of all five kernels on eleven layer
        // shapes x ten batch sizes; their choice is within 1 % of the best measured in total
        // (the two-candidate rule this replaces: 19 % above).
        const double steps = K / 128.0, wbytes = (double)N * K;
        auto rounds = [](double tiles) { return ceil(tiles / 256.0); };
        const double tiles_h = (double)((M + 63) / 64) * ((N + 63) / 64);
        const double tiles_g = (double)((M + 127) / 128) * ((N + 63) / 64);
        const double tiles_t = (double)((M + 127) / 128) * ((N + 127) / 128);
        // up to 192 tiles the idle CUs read the weight through the caches meanwhile (warm_caches):
        // steps measured 13 % (64 x 64) and 20-25 % (the larger tiles) shorter
        auto warmed = [&](double tiles, double f) { return tiles <= 192 && wbytes <= 64.0 * 1048576.0 ? f : 1.0; };
        const double t_h = 2.5 + steps * (0.22 + N * 1.6e-5) * warmed(tiles_h, 0.87) * (1.0 + 0.50 * (rounds(tiles_h) - 1));
        const double t_g = 2.5 + steps * (0.36 + N * 1.2e-5) * warmed(tiles_g, 0.78) * (1.0 + 0.75 * (rounds(tiles_g) - 1));
        const double t_t = 2.5 + steps * (0.50 + N * 1.5e-5) * warmed(tiles_t, 0.78) * (1.0 + 0.65 * (rounds(tiles_t) - 1));
        double t_rows = 1e30;
        if (K <= 10240) {
            const double per_chunk = 0.5 + wbytes / (gemm_w8a8_rows_tiles(N) * 2.0e7);
            t_rows = ((M + 127) / 128) * (3.2 + wbytes / 6.0e6) + ((M + 15) / 16) * per_chunk;
        }
        // Split-K on the 64 x 64 tile where the caller brought room for the partial tiles (the
        // arrival counters cleared): few tiles and many steps, e.g. 64 rows of 9728 -> 2560 are
        // 40 tiles x 76 steps on 40 of 256 CUs.  As many splits as keep one workgroup per CU and
        // four steps per split.  With the whole chip pulling, the steps run into the weight stream
        // (about 5 TB/s in so short a launch), and the hand-over -- partial tiles written through
        // to memory, the arrival, the last workgroup's reads: three trips to memory, the L2s of
        // the XCDs not being coherent with each other -- costs 5 us whatever the shape.
        int splits = 1, splits_g = 1;
        double t_s = 1e30, t_sg = 1e30;
        auto split_count = [&](double tiles) {
            int n = (int)(256.0 / tiles);
            if (n > steps / 4) n = (int)(steps / 4);
            return n > 8 ? 8 : n;
        };
        if (arrivals && partials && tiles_h <= 128) {
            splits = split_count(tiles_h);
            if (splits >= 2 && (size_t)(splits * tiles_h) * 64 * 64 * 4 <= partial_bytes)
                t_s = 2.5 + fmax(ceil(steps / splits) * 0.26, wbytes / 5.0e6) + 5.0;
        }
        // the same on the 128(m) x 64(n) tile (129..256 rows): a step is longer, the hand-over twice the bytes
        if (arrivals && partials && tiles_g <= 128 && M > 128) {
            splits_g = split_count(tiles_g);
            if (splits_g >= 2 && (size_t)(splits_g * tiles_g) * 128 * 64 * 4 <= partial_bytes)
                t_sg = 2.5 + fmax(ceil(steps / splits_g) * 0.42, wbytes / 5.0e6) + 6.0;
        }
        if ((t_s < t_rows && t_s < t_h && t_s < t_g && t_s < t_t) || (t_sg < t_rows && t_sg < t_h && t_sg < t_g && t_sg < t_t)) {
            const bool wide_m = t_sg < t_s;
            Args a;
            a.xq = xq;
            a.wq = wq;
            a.xs = xs;
            a.ws = ws;
            a.y = static_cast<uint16_t *>(y);
            a.acc_out = acc_out;
            a.M = M;
            a.N = N;
            a.K = K;
            a.ldy = ldy;
            a.splits = wide_m ? splits_g : splits;
            a.partials = static_cast<int32_t *>(partials);
            a.arrivals = arrivals;
            return wide_m ? launch_split<1, 2, 3>(a, static_cast<hipStream_t>(stream))
                          : launch_split<1, 1, 4>(a, static_cast<hipStream_t>(stream));
        }
        if (t_rows <= t_h && t_rows <= t_g && t_rows <= t_t) {
            for (int lo = 0; lo < M; lo += 128) {
                const int m = M - lo < 128 ? M - lo : 128;
                const int rc = gemm_w8a8_rows16(xq + (size_t)lo * K, wq, xs + lo, ws,
                                                static_cast<uint16_t *>(y) + (size_t)lo * ldy,
                                                acc_out ? acc_out + (size_t)lo * N : nullptr, m, N, K, ldy, stream);
                if (rc != CMI_OK) return rc == CMI_E_UNSUPPORTED ? fail(rc, "cmi_gemm_w8a8: internal dispatch") : rc;
            }
            return CMI_OK;
        }
        mid = t_h <= t_g && t_h <= t_t ? 6464 : t_g <= t_t ? 64 : 128;
    }
    if (K % BK != 0 || N < 8) return gemm_w8a8_generic(xq, wq, xs, ws, y, acc_out, M, N, K, ldy, stream);
    Args a;
    a.xq = xq;
    a.wq = wq;
    a.xs = xs;
    a.ws = ws;
    a.y = static_cast<uint16_t *>(y);
    a.acc_out = acc_out;
    a.M = M;
    a.N = N;
    a.K = K;
    a.ldy = ldy;
    a.splits = 1;
    a.partials = nullptr;
    a.arrivals = nullptr;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // Tile choice above 256 rows.  Every tile kernel is a chain of K / 128 dependent steps whose
    // length is set by the operand bytes a workgroup pulls per step (it grows with the tile and,
    // the weight being cold, with N) and by how many workgroups share a CU; larger tiles move
    // fewer bytes per MFMA, smaller ones fill the 256 CUs more evenly.  Cost models (us) of the
    // same form as for 17..256 rows, fitted to cold-weight measurements of every kernel on
    // sixteen layer shapes x eleven batch sizes (272..8192 rows): their choice is 0.3 % above the
    // best measured in total, the fill-and-area rule this replaces 2.4 % (and up to 40 % on
    // single shapes, e.g. 2048 x 9728 -> 2560: 84 -> 63 us).
    // CMI_GEMM_TILE=64|128|192|256|320 overrides the tile along n (tests, tuning); 128192 forces
    // 128(n) x 192(m), 6464 the 64 x 64 tile of the mid-batch route.
    int pick;  // 64, 128, 192, 256 or 320: block tile along n; 128192; 6464
    if (force || mid) {
        pick = force ? force : mid;
    } else {
        const double steps = K / 128.0;
        auto cost = [&](int bm, int bn, double a0, double b0, double c0) {
            const double tiles = (double)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
            // the 4-wavefront tiles on up to 192 CUs: the idle CUs warm the caches (see above)
            const double warmed = bm <= 192 && tiles <= 192 && (double)N * K <= 64.0 * 1048576.0 ? 0.8 : 1.0;
            return 2.5 + steps * (a0 + b0 * N) * warmed * (1.0 + c0 * (ceil(tiles / 256.0) - 1.0));
        };
        const struct { int pick; double us; } candidates[] = {
            {64, N > 64 ? cost(128, 64, 0.407, 5.54e-6, 0.796) : 1e30},
            {128, cost(128, 128, 0.555, 9.82e-6, 0.91)},
            {192, cost(128, 192, 0.723, 1.89e-5, 1.03)},
            {128192, cost(192, 128, 0.709, 1.19e-5, 1.12)},
            {256, cost(256, 256, 1.29, 2.33e-5, 1.28)},
            {320, cost(256, 320, 1.60, 3.39e-5, 1.13)},
        };
        pick = 128;
        double best = 1e30;
        for (const auto &c : candidates)
            if (c.us < best) best = c.us, pick = c.pick;
        // Split-K on the 128 x 128 tile where the caller brought room for the partial tiles: a long,
        // narrow projection (9728 -> 2560 at 257..512 rows: 60..80 tiles x 76 steps) leaves most
        // of the CUs idle for a long chain of steps (quantiser + GEMM 38..42 -> 30..34.5 us).  Model
        // as for the smaller tiles; the hand-over moves 64 KiB per workgroup.
        const int tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
        if (arrivals && partials && tiles128 <= 128 && steps >= 16) {
            int splits = 256 / tiles128;
            if (splits > steps / 4) splits = (int)(steps / 4);
            if (splits > 8) splits = 8;
            const double t_split = 2.5 + fmax(ceil(steps / splits) * (0.554 + 1.11e-5 * N), (double)N * K / 5.0e6) + SPLIT128_HANDOVER_US;
            if (splits >= 2 && (size_t)splits * tiles128 * 128 * 128 * 4 <= partial_bytes && t_split < best) {
                a.splits = splits;
                a.partials = static_cast<int32_t *>(partials);
                a.arrivals = arrivals;
                return launch_split<2, 2, 3>(a, st);
            }
        }
    }
    // the 256 x 320 tile: the tile-wise kernel (within 1 % of the two-stage one on the large shapes,
    // 7 % faster at 2048 x 4096 x 2560); a forced 320 still names the two-stage kernel
    // The persistent form (322) keeps its pipeline running from tile to tile -- and takes the same time
    // as the one-tile kernel: at the clock the power limit leaves these launches, closing the gaps
    // between tiles is paid back in clock.  Alternating replays of the two, cold weights, medians:
    // 8192 x 9728 x 2560 (3.9 tiles per CU) 178.0 / 177.9 us, 8192 x 19456 x 2560 (7.6) 372.4 / 371.5 and,
    // in the other order, 359.3 / 356.4; 4096 x 9728 92.5 / 93.5; a single tile 49.3 / 51.1.  (A first
    // comparison read -2 %: there the persistent kernel always ran behind the one-tile kernel and that
    // one behind the slower 256 x 256 kernel, and what a launch follows moves it by more than that.)
    // Kept for study under its code; the library's choice stays the one-tile kernel.
    if (pick == 322) return launch_wide_persistent(a, st);
    if (pick == 321 || (pick == 320 && !force)) return launch_wide_tilewise(a, st);
    if (pick == 320) return launch_wide(a, st);
    if (pick == 256) return launch_big(a, st);
    if (pick == 192) return launch<3, 2, 3>(a, st);
    if (pick == 128192) return launch<2, 3, 3>(a, st);
    // 64 x 64 tiles, four LDS stages (more stages measured the same): half the bytes per step and
    // twice the workgroups of the 128 x 64 tile for batches of up to 64 rows or few n tiles
    if (pick == 6464) return launch<1, 1, 4>(a, st);
    if (pick == 64) {
        // 128(m) x 64(n): twice the workgroups of the 128 x 128 tile with half the MFMAs per
        // dependent step each
        const int tiles64 = ((M + 127) / 128) * ((N + 63) / 64);
        if (tiles64 <= 256) return launch<1, 2, 3>(a, st);
        return launch<1, 2, 2>(a, st);
    }
    // Up to one 128 x 128 workgroup per CU a third LDS stage (96 KiB, one workgroup per CU anyway)
    // puts two steps of loads in flight (-20 % at K = 2560, -33 % at K = 9728); with two
    // workgroups per CU it measured slower.
    const int tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
    if (tiles128 <= 256) return launch<2, 2, 3>(a, st);
    return launch<2, 2, 2>(a, st);
}
