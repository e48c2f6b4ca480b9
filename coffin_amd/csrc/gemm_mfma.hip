// Prefill GEMMs on CDNA4 int8 MFMA: W8A8 (int8 weights) and W4A8 (group-128 int4
// weights), both against per-token int8 activations, scales fused in.
//
//   W8A8: acc[m,n] = sum_k xq[m,k]*wq[n,k]          int32, exact
//         y[m,n]   = bf16((float)acc * xs[m] * ws[n])    left to right, one narrowing
//   W4A8: sum_g    = sum_{k in g} xq[m,k]*(code-8)  int32, exact, per group of 128
//         total    = fma((float)sum_g, ws[n,g], total)   g ascending from 0.f
//         y[m,n]   = bf16(total * xs[m])
//
// Both operands are K-contiguous ([M,K] activations, [N,K] weights), which is
// the layout v_mfma_i32_16x16x64_i8 wants: a lane feeds 16 consecutive k bytes
// of one row.  The weight supplies the MFMA rows and the activation the MFMA
// columns, so a lane ends up with four consecutive n of one m and stores 8
// contiguous bytes of y.
//
// Tiling: workgroup = 4 wavefronts (2 x 2), block tile 128(m) x 128(n) x 128
// bytes of k, wavefront tile 64 x 64 = 4 x 4 MFMA tiles, accumulators in
// registers for the whole K loop.  Tiles are staged global -> registers -> LDS
// (rows padded by 16 B so that 8 consecutive rows land in 8 distinct 16-byte
// bank groups), double buffered: the next k tile is fetched from HBM/L2 while
// the current one is multiplied.  int4 weights are widened to int8 on their
// way into LDS (half the HBM bytes, same inner loop) and one k tile is exactly
// one scale group, so the group flush sits at the k-tile boundary.  Workgroup
// ids are remapped so that each of the 8 XCDs (private L2 each) works on a
// contiguous band of n tiles.
#include "common.hpp"
#include "gemm_tiles.hpp"

namespace {

using namespace cmi;

constexpr int BM = 128;  // activation rows per block
constexpr int BN = 128;  // weight rows per block
constexpr int BK = 128;  // k elements (= int8 bytes) per stage; one int4 scale group
constexpr int PAD = 16;
constexpr int LDS_STRIDE = BK + PAD;          // 144 = 9 * 16
constexpr int TILE_BYTES = 128 * LDS_STRIDE;  // one operand, one stage
constexpr int STAGE_BYTES = 2 * TILE_BYTES;
constexpr int THREADS = 256;
constexpr int CHUNKS_PER_ROW = BK / 16;                // 8
constexpr int LOADS8 = 128 * CHUNKS_PER_ROW / THREADS; // 4 x 16 B per thread (int8 operand)
constexpr int LOADS4 = LOADS8 / 2;                     // 2 x 16 B per thread (int4 operand)
constexpr int WS_BYTES = 2 * BN * 4;                   // W4A8: two stages of group scales

struct GemmArgs {
    const int8_t *xq;
    const void *w;     // int8 [N,K] or re-laid-out int4 [N,K/2]
    const float *xs;
    const float *ws;   // W8A8: [N]; W4A8: [N, K/128]
    uint16_t *y;
    int32_t *acc_out;  // W8A8: [M,N]; W4A8: [M, K/128, N]; nullable
    int M, N, K, ldy, G;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ void fetch_i8(const int8_t *base, int rows, int K, int row0, int k0,
                                         uint4 (&reg)[LOADS8]) {
#pragma unroll
    for (int i = 0; i < LOADS8; ++i) {
        const int c = threadIdx.x + i * THREADS;
        const int r = c / CHUNKS_PER_ROW, kc = c % CHUNKS_PER_ROW;
        int row = row0 + r;
        row = row < rows ? row : rows - 1;
        const int k = k0 + kc * 16;
        reg[i] = k < K ? *reinterpret_cast<const uint4 *>(base + (size_t)row * K + k)
                       : make_uint4(0, 0, 0, 0);
    }
}

__device__ __forceinline__ void stash_i8(int8_t *lds, const uint4 (&reg)[LOADS8]) {
#pragma unroll
    for (int i = 0; i < LOADS8; ++i) {
        const int c = threadIdx.x + i * THREADS;
        const int r = c / CHUNKS_PER_ROW, kc = c % CHUNKS_PER_ROW;
        *reinterpret_cast<uint4 *>(lds + r * LDS_STRIDE + kc * 16) = reg[i];
    }
}

// int4: a 16-byte chunk carries 32 k; four chunks per row and k tile.
__device__ __forceinline__ void fetch_i4(const uint8_t *base, int rows, int K, int row0, int k0,
                                         uint4 (&reg)[LOADS4]) {
#pragma unroll
    for (int i = 0; i < LOADS4; ++i) {
        const int c = threadIdx.x + i * THREADS;
        const int r = c / 4, kc = c % 4;
        int row = row0 + r;
        row = row < rows ? row : rows - 1;
        const int k = k0 + kc * 32;
        reg[i] = k < K ? *reinterpret_cast<const uint4 *>(base + ((size_t)row * K + k) / 2)
                       : make_uint4(0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u);
    }
}

__device__ __forceinline__ void stash_i4(int8_t *lds, const uint4 (&reg)[LOADS4]) {
#pragma unroll
    for (int i = 0; i < LOADS4; ++i) {
        const int c = threadIdx.x + i * THREADS;
        const int r = c / 4, kc = c % 4;
        const uint32_t w[4] = {reg[i].x, reg[i].y, reg[i].z, reg[i].w};
        uint4 lo, hi;  // k 0..15 and 16..31 of the chunk
        widen_w4_piece(w[0], w[1], w[2], w[3], lo, hi);
        int8_t *dst = lds + r * LDS_STRIDE + kc * 32;
        *reinterpret_cast<uint4 *>(dst) = lo;
        *reinterpret_cast<uint4 *>(dst + 16) = hi;
    }
}

template <bool W4>
__global__ void __launch_bounds__(THREADS)
gemm_kernel(const GemmArgs a) {
    extern __shared__ __align__(16) int8_t lds[];  // [2 stages][W tile | X tile] (+ W4 scales)
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wn = wave & 1, wm = wave >> 1;

    // XCD-aware tile order: hardware deals workgroups round-robin to the 8
    // XCDs; give XCD x the logical tiles [x*per, (x+1)*per) so that its L2
    // keeps a contiguous band of weight rows, m fastest inside the band.
    const int total_tiles = a.tiles_m * a.tiles_n;
    int tile = blockIdx.x;
    if (total_tiles % 8 == 0) tile = (blockIdx.x % 8) * (total_tiles / 8) + blockIdx.x / 8;
    const int tn = tile / a.tiles_m, tm = tile - tn * a.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    v4i32 acc[4][4];  // [n tile][m tile]
    float total[W4 ? 4 : 1][W4 ? 4 : 1][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[i][j] = v4i32{0, 0, 0, 0};
            if constexpr (W4) {
#pragma unroll
                for (int r = 0; r < 4; ++r) total[i][j][r] = 0.f;
            }
        }

    float *wsl = reinterpret_cast<float *>(lds + 2 * STAGE_BYTES);  // W4: [2][BN]
    const int8_t *w8 = static_cast<const int8_t *>(a.w);
    const uint8_t *w4 = static_cast<const uint8_t *>(a.w);

    uint4 wreg[W4 ? LOADS4 : LOADS8], xreg[LOADS8];
    float wsreg = 0.f;
    const int ws_row = n0 + (int)threadIdx.x < a.N ? n0 + (int)threadIdx.x : a.N - 1;
    if constexpr (W4) {
        fetch_i4(w4, a.N, a.K, n0, 0, wreg);
        if (threadIdx.x < BN) wsreg = a.ws[(size_t)ws_row * a.G];
    } else {
        fetch_i8(w8, a.N, a.K, n0, 0, wreg);
    }
    fetch_i8(a.xq, a.M, a.K, m0, 0, xreg);
    if constexpr (W4) {
        stash_i4(lds, wreg);
        if (threadIdx.x < BN) wsl[threadIdx.x] = wsreg;
    } else {
        stash_i8(lds, wreg);
    }
    stash_i8(lds + TILE_BYTES, xreg);
    __syncthreads();

    const int frag_row = lane & 15, frag_k = (lane >> 4) * 16;
    const int mcol = lane & 15, nquad = (lane >> 4) * 4;
    const int ksteps = (a.K + BK - 1) / BK;
    for (int ks = 0; ks < ksteps; ++ks) {
        const int cur = ks & 1;
        const bool more = ks + 1 < ksteps;
        if (more) {
            if constexpr (W4) {
                fetch_i4(w4, a.N, a.K, n0, (ks + 1) * BK, wreg);
                if (threadIdx.x < BN) wsreg = a.ws[(size_t)ws_row * a.G + ks + 1];
            } else {
                fetch_i8(w8, a.N, a.K, n0, (ks + 1) * BK, wreg);
            }
            fetch_i8(a.xq, a.M, a.K, m0, (ks + 1) * BK, xreg);
        }
        const int8_t *wt = lds + cur * STAGE_BYTES + (wn * 64 + frag_row) * LDS_STRIDE + frag_k;
        const int8_t *xt = lds + cur * STAGE_BYTES + TILE_BYTES + (wm * 64 + frag_row) * LDS_STRIDE + frag_k;
#pragma unroll
        for (int kk = 0; kk < BK / 64; ++kk) {
            v4i32 wf[4], xf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                wf[i] = *reinterpret_cast<const v4i32 *>(wt + i * 16 * LDS_STRIDE + kk * 64);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                xf[j] = *reinterpret_cast<const v4i32 *>(xt + j * 16 * LDS_STRIDE + kk * 64);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[i], xf[j], acc[i][j], 0, 0, 0);
        }
        if constexpr (W4) {
            // End of scale group ks: fold the int32 sums into the fp32 totals.
            const float *wsc = wsl + cur * BN + wn * 64 + nquad;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 sc = *reinterpret_cast<const float4 *>(wsc + i * 16);
                const float scv[4] = {sc.x, sc.y, sc.z, sc.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int vals[4] = {acc[i][j].x, acc[i][j].y, acc[i][j].z, acc[i][j].w};
                    if (a.acc_out) {
                        const int m = m0 + wm * 64 + j * 16 + mcol;
                        const int n = n0 + wn * 64 + i * 16 + nquad;
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (m < a.M && n + r < a.N)
                                a.acc_out[((size_t)m * a.G + ks) * a.N + n + r] = vals[r];
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        total[i][j][r] = fmaf((float)vals[r], scv[r], total[i][j][r]);
                    acc[i][j] = v4i32{0, 0, 0, 0};
                }
            }
        }
        if (more) {
            int8_t *nxt = lds + (cur ^ 1) * STAGE_BYTES;
            if constexpr (W4) {
                stash_i4(nxt, wreg);
                if (threadIdx.x < BN) wsl[(cur ^ 1) * BN + threadIdx.x] = wsreg;
            } else {
                stash_i8(nxt, wreg);
            }
            stash_i8(nxt + TILE_BYTES, xreg);
        }
        __syncthreads();
    }

    // Epilogue: lane holds n = nb + 4*(lane/16) + r (r = 0..3) for m = mb + lane%16.
    const bool vec_ok = (a.ldy % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.y) & 7) == 0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int m = m0 + wm * 64 + j * 16 + mcol;
        if (m >= a.M) continue;
        const float xm = a.xs[m];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + wn * 64 + i * 16 + nquad;
            if (n >= a.N) continue;
            uint32_t o[4];
            if constexpr (W4) {
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = f32_to_bf16_bits(total[i][j][r] * xm);
            } else {
                const int vals[4] = {acc[i][j].x, acc[i][j].y, acc[i][j].z, acc[i][j].w};
                if (a.acc_out) {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (n + r < a.N) a.acc_out[(size_t)m * a.N + n + r] = vals[r];
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float wsn = n + r < a.N ? a.ws[n + r] : 0.f;
                    const float t = (float)vals[r] * xm;
                    o[r] = f32_to_bf16_bits(t * wsn);
                }
            }
            uint16_t *dst = a.y + (size_t)m * a.ldy + n;
            if (vec_ok && n + 3 < a.N) {
                uint2 pk;
                pk.x = o[0] | (o[1] << 16);
                pk.y = o[2] | (o[3] << 16);
                *reinterpret_cast<uint2 *>(dst) = pk;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < a.N) dst[r] = (uint16_t)o[r];
            }
        }
    }
}

template <bool W4>
int launch(GemmArgs &a, hipStream_t st, const char *what) {
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (a.N + BN - 1) / BN;
    const size_t lds = 2 * STAGE_BYTES + (W4 ? WS_BYTES : 0);
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemm_kernel<W4>),
                                   (int)lds, devices, what))
        return rc;
    gemm_kernel<W4><<<dim3(a.tiles_m * a.tiles_n), dim3(THREADS), lds, st>>>(a);
    return check_launch(what);
}

}  // namespace

// Register-staged W8A8 kernel: any K that is a multiple of 16 (arguments already validated).
int cmi::gemm_w8a8_generic(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws,
                           void *y, int32_t *acc_out, int M, int N, int K, int ldy, void *stream) {
    GemmArgs a;
    a.xq = xq;
    a.w = wq;
    a.xs = xs;
    a.ws = ws;
    a.y = static_cast<uint16_t *>(y);
    a.acc_out = acc_out;
    a.M = M;
    a.N = N;
    a.K = K;
    a.ldy = ldy;
    a.G = 1;
    return launch<false>(a, static_cast<hipStream_t>(stream), "cmi_gemm_w8a8");
}
