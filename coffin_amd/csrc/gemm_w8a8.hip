// W8A8 prefill GEMM, software-pipelined for CDNA4 int8 MFMA (K a multiple of 128).
//
//   acc[m,n] = sum_k xq[m,k] * wq[n,k]           int32, exact
//   y[m,n]   = bf16((float)acc * xs[m] * ws[n])   left to right, one narrowing
//
// v_mfma_i32_32x32x32_i8 (one wavefront per SIMD already sustains ~90 % of the
// int8 peak with it; the 16x16x64 form needs two) with the weight on the MFMA
// rows and the activation on the MFMA columns, both K-contiguous in memory
// (16 consecutive k per lane), so a lane ends with groups of four consecutive n
// of one m.
//
// Workgroup = 4 wavefronts (2 x 2), block tile 128(m) x 128(n), wavefront tile
// 64 x 64 = 2 x 2 MFMA tiles held in registers for the whole K loop.  K is walked
// in steps of 128 (one whole cache line per row: with 64-byte steps every line
// was fetched from L2 twice, the L1 being too small to keep it for a step)
// through two LDS stages filled by direct global -> LDS loads
// (global_load_lds_dwordx4: no staging registers); the register copy of the
// current fragments acts as the third stage.  Two workgroups share a CU.  A direct load lays the 64 lanes' 16-byte chunks out
// contiguously, so the bank-conflict-free arrangement is made on the global
// side: lane i of a load fetches the chunk that belongs at LDS slot i, with the
// chunk index XOR-swizzled by (row / 2) % 8.  Sixteen consecutive lanes of a
// fragment read (16 rows, one k chunk) then touch 16 distinct 16-byte slots of
// the 256-byte bank row.  Fragments for step s+1 are read from LDS while the 8
// MFMAs of step s issue.  The epilogue goes through LDS once more so that every
// lane stores 16 contiguous bytes of y.
// One s_barrier per step, with explicit vmcnt/lgkmcnt waits (a __syncthreads
// would drain the whole prefetch ring).  Workgroup ids are remapped so each of
// the 8 XCDs (private L2) owns a contiguous band of n tiles.
#include "common.hpp"

namespace {

using namespace cmi;

constexpr int BM = 128, BN = 128, BK = 128;   // BK = one 128-byte cache line per row and step
constexpr int STAGES = 2;
constexpr int THREADS = 256;
constexpr int TILE_BYTES = 128 * BK;            // one operand, one stage: 16 KiB
constexpr int STAGE_BYTES = 2 * TILE_BYTES;     // W tile then X tile
constexpr int LDS_BYTES = STAGES * STAGE_BYTES; // 64 KiB: two workgroups per CU

struct Args {
    const int8_t *xq;
    const int8_t *wq;
    const float *xs;
    const float *ws;
    uint16_t *y;
    int32_t *acc_out;
    int M, N, K, ldy;
    int tiles_m, tiles_n;
};

typedef __attribute__((address_space(3))) void *lds_ptr_t;

__global__ void __launch_bounds__(THREADS)
gemm_w8a8_pipe_kernel(const Args a) {
    extern __shared__ __align__(16) int8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wn = wave & 1, wm = wave >> 1;

    // XCD-aware tile order: workgroups are dealt round-robin to the 8 XCDs; XCD x
    // gets logical tiles [x*per, (x+1)*per), m fastest inside a band of n tiles.
    const int total = a.tiles_m * a.tiles_n;
    int tile = blockIdx.x;
    if (total % 8 == 0) tile = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;
    const int tn = tile / a.tiles_m, tm = tile - tn * a.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    // Global side of the direct loads.  One load instruction moves 8 rows x 128 B
    // (whole cache lines) into 1 KiB of LDS; a wavefront fills row groups
    // 4*wave .. 4*wave+3 of both tiles.  Lane i lands in slot i of the group:
    // row = i/8, stored chunk = i%8, which holds k chunk (i%8) ^ ((row/2) % 8).
    const int lrow = lane >> 3;
    const int8_t *wsrc[4], *xsrc[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int row = (4 * wave + g) * 8 + lrow;
        const int kc = (lane & 7) ^ ((row >> 1) & 7);
        const int nrow = min(n0 + row, a.N - 1), mrow = min(m0 + row, a.M - 1);
        wsrc[g] = a.wq + (size_t)nrow * a.K + kc * 16;
        xsrc[g] = a.xq + (size_t)mrow * a.K + kc * 16;
    }
    auto issue = [&](int stage, int ks) {
        int8_t *base = lds + stage * STAGE_BYTES + (4 * wave) * 1024;
        const int k = ks * BK;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            __builtin_amdgcn_global_load_lds((const void *)(wsrc[g] + k),
                                             (lds_ptr_t)(base + g * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const void *)(xsrc[g] + k),
                                             (lds_ptr_t)(base + TILE_BYTES + g * 1024), 16, 0, 0);
        }
    };

    // LDS side: lane reads row (lane%32) of a 32-row MFMA tile; for k quarter q
    // (32 k each) its 16 bytes are k chunk 2q + lane/32.
    const int frow = lane & 31;
    const int fsw = (frow >> 1) & 7;
    int foff[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) foff[q] = frow * BK + ((2 * q + (lane >> 5)) ^ fsw) * 16;
    // frag[t][q]: MFMA tile t (0..1), k quarter q (0..3)
    auto read_frags = [&](int stage, v4i32 (&wf)[2][4], v4i32 (&xf)[2][4]) {
        const int8_t *wt = lds + stage * STAGE_BYTES + wn * 64 * BK;
        const int8_t *xt = lds + stage * STAGE_BYTES + TILE_BYTES + wm * 64 * BK;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                wf[t][q] = *reinterpret_cast<const v4i32 *>(wt + t * 32 * BK + foff[q]);
                xf[t][q] = *reinterpret_cast<const v4i32 *>(xt + t * 32 * BK + foff[q]);
            }
    };

    v16i32 acc[2][2];  // [n tile][m tile]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    auto mma = [&](const v4i32 (&wf)[2][4], const v4i32 (&xf)[2][4]) {
#pragma unroll
        for (int h = 0; h < 4; ++h)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i][h], xf[j][h], acc[i][j], 0, 0, 0);
    };

    const int ksteps = a.K / BK;
    // One pipeline step.  Stage ks%2 was emptied into registers during step ks-1,
    // so once every wavefront is past the barrier it takes the loads of step ks+2;
    // stage (ks+1)%2 has landed (it was requested a whole step ago) and its
    // fragments are read while the 16 MFMAs of step ks issue.
    auto step = [&](int ks, const v4i32 (&cw)[2][4], const v4i32 (&cx)[2][4], v4i32 (&nw)[2][4],
                    v4i32 (&nx)[2][4]) {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (ks + 2 < ksteps) issue(ks % STAGES, ks + 2);
        if (ks + 1 < ksteps) read_frags((ks + 1) % STAGES, nw, nx);
        mma(cw, cx);
    };

    issue(0, 0);
    if (ksteps > 1) issue(1, 1);
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");   // stage 0 (8 loads per stage and wavefront)
    if (ksteps == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    v4i32 w0[2][4], x0[2][4], w1[2][4], x1[2][4];
    read_frags(0, w0, x0);
    int ks = 0;
    for (; ks + 1 < ksteps; ks += 2) {
        step(ks, w0, x0, w1, x1);
        step(ks + 1, w1, x1, w0, x0);
    }
    if (ks < ksteps) step(ks, w0, x0, w1, x1);

    // Epilogue.  Accumulator element v of tile (i, j) in lane l is
    //   n = nb + 32*i + 8*(v/4) + 4*(l/32) + v%4,   m = mb + 32*j + l%32.
    // Scale, narrow, park the wavefront's 64 x 64 bf16 tile in LDS (row = m,
    // 144-byte pitch), then write rows back 16 bytes per lane.
    if (a.acc_out) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int m = m0 + wm * 64 + j * 32 + (lane & 31);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int n = n0 + wn * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                    if (m < a.M && n < a.N) a.acc_out[(size_t)m * a.N + n] = acc[i][j][v];
                }
            }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();  // every wavefront is done reading operand stages
    asm volatile("" ::: "memory");
    constexpr int PITCH = 144;     // 64 bf16 + 16 B: 8 rows -> 8 distinct 16-byte bank groups
    int8_t *park = lds + wave * (64 * PITCH);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int ml = j * 32 + (lane & 31);
        const int m = m0 + wm * 64 + ml;
        const float xm = a.xs[min(m, a.M - 1)];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nl = i * 32 + 8 * q + 4 * (lane >> 5);
                const int n = n0 + wn * 64 + nl;
                const float4 sc = *reinterpret_cast<const float4 *>(a.ws + min(n, a.N - 4));
                const float scv[4] = {sc.x, sc.y, sc.z, sc.w};
                uint32_t o[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    // ws index is clamped for the ragged edge; those columns are never stored
                    const float wsn = n + 3 < a.N ? scv[r] : a.ws[min(n + r, a.N - 1)];
                    const float t = (float)acc[i][j][4 * q + r] * xm;
                    o[r] = f32_to_bf16_bits(t * wsn);
                }
                uint2 pk;
                pk.x = o[0] | (o[1] << 16);
                pk.y = o[2] | (o[3] << 16);
                *reinterpret_cast<uint2 *>(park + ml * PITCH + nl * 2) = pk;
            }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own tile only: no barrier needed
    const bool vec_ok = (a.ldy % 8 == 0) && ((reinterpret_cast<uintptr_t>(a.y) & 15) == 0);
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const int ml = p * 8 + (lane >> 3), c = lane & 7;  // 8 lanes x 16 B = one 64-wide row
        const int m = m0 + wm * 64 + ml;
        const int n = n0 + wn * 64 + c * 8;
        if (m >= a.M || n >= a.N) continue;
        const uint4 v = *reinterpret_cast<const uint4 *>(park + ml * PITCH + c * 16);
        uint16_t *dst = a.y + (size_t)m * a.ldy + n;
        if (vec_ok && n + 7 < a.N) {
            *reinterpret_cast<uint4 *>(dst) = v;
        } else {
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int r = 0; r < 8; ++r)
                if (n + r < a.N) dst[r] = (uint16_t)(w[r >> 1] >> ((r & 1) * 16));
        }
    }
}

}  // namespace

extern "C" int cmi_gemm_w8a8(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws,
                             void *y, int32_t *acc_out, int M, int N, int K, int ldy,
                             void *stream) {
    CMI_REQUIRE(M >= 0 && N >= 1 && K >= 16, CMI_E_ARG, "cmi_gemm_w8a8: bad shape M=%d N=%d K=%d", M, N, K);
    if (M == 0) return CMI_OK;  // an empty batch has no storage to point at
    CMI_REQUIRE(xq && wq && xs && ws && y, CMI_E_ARG, "cmi_gemm_w8a8: null pointer");
    CMI_REQUIRE(ldy >= N, CMI_E_ARG, "cmi_gemm_w8a8: ldy=%d is smaller than N=%d", ldy, N);
    CMI_REQUIRE(K % 16 == 0, CMI_E_UNSUPPORTED, "cmi_gemm_w8a8: K=%d is not a multiple of 16", K);
    CMI_REQUIRE(aligned(xq, 16) && aligned(wq, 16), CMI_E_ARG,
                "cmi_gemm_w8a8: xq and wq must be 16-byte aligned");
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
    a.tiles_m = (M + BM - 1) / BM;
    a.tiles_n = (N + BN - 1) / BN;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_w8a8_pipe_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess)
            return fail(CMI_E_HIP, "cmi_gemm_w8a8: cannot reserve %d bytes of LDS", LDS_BYTES);
        configured = true;
    }
    gemm_w8a8_pipe_kernel<<<dim3(a.tiles_m * a.tiles_n), dim3(THREADS), LDS_BYTES,
                            static_cast<hipStream_t>(stream)>>>(a);
    return check_launch("cmi_gemm_w8a8");
}
