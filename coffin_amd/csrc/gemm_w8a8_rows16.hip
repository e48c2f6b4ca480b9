// W8A8 projection for 1..16 (and, weight kept in registers, up to 128) activation rows: the weight is
// read once, straight into registers, and the kernel is HBM-bound like a GEMV.
//
//   acc[m,n] = sum_k xq[m,k] * wq[n,k]                  int32, exact
//   y[m,n]   = bf16(((float)acc * xs[m]) * ws[n])
//
// The tiled GEMM kernels spend a 128-row tile on such a batch.  Here a workgroup
// owns 16 weight rows and one v_mfma_i32_16x16x64_i8 covers them against all 16
// activation rows for 64 k: lane l supplies bytes 64*s + 16*(l/16) .. +15 of
// weight row l%16 and the same bytes of activation row l%16.  The wavefronts of
// the workgroup split K by 128-byte lines (wavefront w takes lines w, w+WAVES,
// ..), request all their bytes before anything else -- as whole cache lines,
// rearranged for the MFMA through a private LDS patch -- and add their int32
// partial tiles through LDS (integer sums: order does not matter).  Thread
// (n, m) then applies the two scales.
#include "rows16_tile.hpp"

namespace {

using namespace cmi;
using namespace cmi::rows16;

constexpr int ROWS = 16;
constexpr int LINE = 128;  // bytes of one weight row per line = 2 MFMA steps

struct Args {
    const int8_t *xq, *wq;
    const float *xs, *ws;
    uint16_t *y;
    int32_t *acc_out;
    int M, N, K, ldy;
};

// NLP: lines per wavefront (upper bound; surplus slots are skipped).  WAVES: 4 or 8.
template <int NLP, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
gemm_w8a8_rows16_kernel(const Args a) {
    __shared__ __align__(16) int32_t partial[WAVES][64][4];
    __shared__ __align__(16) uint8_t patches[WAVES][PATCH_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = lane >> 4;
    const int n0 = blockIdx.x * ROWS;
    const int lines = a.K / LINE;
    uint8_t *patch = patches[wave];

    // activations first (L2 resident; memory answers in request order), then every weight byte
    v4i32 xr[NLP][2], wr[NLP][2];
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
        const int line = wave + i * WAVES;
        if (line >= lines) break;  // uniform per wavefront
#pragma unroll
        for (int h = 0; h < 2; ++h)  // rows past M repeat the last one; their sums are dropped
            xr[i][h] = *reinterpret_cast<const v4i32 *>(a.xq + tile_src(lane, h, 0, a.M - 1, a.K, line * LINE));
    }
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
        const int line = wave + i * WAVES;
        if (line >= lines) break;
#pragma unroll
        for (int h = 0; h < 2; ++h)
            wr[i][h] = __builtin_nontemporal_load(
                reinterpret_cast<const v4i32 *>(a.wq + tile_src(lane, h, n0, a.N - 1, a.K, line * LINE)));
    }

    // the scales of the output this thread will finish, requested behind the operands: asked for at
    // the end they are cold loads under a saturated memory system
    const float ws_out = a.ws[min(n0 + (int)((threadIdx.x >> 2) & 15), a.N - 1)];
    const float xs_out = a.xs[min((int)(4 * ((threadIdx.x >> 6) & 3) + (threadIdx.x & 3)), a.M - 1)];

    // into the MFMA arrangement (lane: row lane%16, pieces kq and 4+kq), then the products;
    // the accumulator of lane l holds (n = l%16, m = 4*kq + v), v = 0..3
    v4i32 acc = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
        const int line = wave + i * WAVES;
        if (line >= lines) break;
        tile_park(patch, lane, xr[i][0], xr[i][1]);
        xr[i][0] = tile_take(patch, lane, kq);
        xr[i][1] = tile_take(patch, lane, 4 + kq);
    }
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
        const int line = wave + i * WAVES;
        if (line >= lines) break;
        tile_park(patch, lane, wr[i][0], wr[i][1]);
        const v4i32 w0 = tile_take(patch, lane, kq), w1 = tile_take(patch, lane, 4 + kq);
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xr[i][0], w0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xr[i][1], w1, acc, 0, 0, 0);
    }
    *reinterpret_cast<v4i32 *>(&partial[wave][lane][0]) = acc;
    __syncthreads();

    if (threadIdx.x < 256) {
        const int l = threadIdx.x >> 2, v = threadIdx.x & 3;
        const int n = n0 + (l & 15), m = 4 * (l >> 4) + v;
        if (n < a.N && m < a.M) {
            int s = 0;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) s += partial[wv][l][v];
            if (a.acc_out) a.acc_out[(size_t)m * a.N + n] = s;
            a.y[(size_t)m * a.ldy + n] = (uint16_t)f32_to_bf16_bits(((float)s * xs_out) * ws_out);
        }
    }
}

template <int NLP, int WAVES>
int launch(const Args &a, hipStream_t st) {
    const dim3 grid((a.N + ROWS - 1) / ROWS);
    gemm_w8a8_rows16_kernel<NLP, WAVES><<<grid, dim3(WAVES * 64), 0, st>>>(a);
    return check_launch("cmi_gemm_w8a8");
}


// 17..128 activation rows: the workgroup's T tiles of 16 weight rows are asked for once and stay in
// registers in the MFMA arrangement; the activation rows go through in chunks of 16, each fetched
// tile serving all T weight tiles (every workgroup reads all of xq through L2: M * K bytes times
// N / (16 T) workgroups, which at T = 1 is four times the weight bytes for 64 rows).  Integer
// sums are exact in any order, so the wavefronts add their partial tiles into one LDS tile per
// chunk with ds_add and the bits are those of the 16-row kernel by construction.
constexpr int MAX_CHUNKS = 8;

template <int NLP, int WAVES, int T>
__global__ void __launch_bounds__(WAVES * 64)
gemm_w8a8_rows128_kernel(const Args a) {
    __shared__ __align__(16) int32_t sums[MAX_CHUNKS * T][64][4];
    __shared__ __align__(16) uint8_t patches[WAVES][PATCH_BYTES];
    __shared__ float ws_tile[T * ROWS], xs_tile[MAX_CHUNKS * ROWS];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = lane >> 4;
    const int n0 = blockIdx.x * (ROWS * T);
    const int lines = a.K / LINE;
    const int chunks = (a.M + ROWS - 1) / ROWS;
    uint8_t *patch = patches[wave];
    auto line_of = [&](int i) { return min(wave + i * WAVES, lines - 1); };  // surplus slots repeat the last line

    v4i32 xr[NLP][2], wr[T][NLP][2];
    auto request_x = [&](int c, int i) {
#pragma unroll
        for (int h = 0; h < 2; ++h)  // rows past M repeat the last one; their sums are dropped
            xr[i][h] = *reinterpret_cast<const v4i32 *>(
                a.xq + tile_src(lane, h, c * ROWS, a.M - 1, a.K, line_of(i) * LINE));
    };
#pragma unroll
    for (int i = 0; i < NLP; ++i) request_x(0, i);
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int i = 0; i < NLP; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                wr[t][i][h] = __builtin_nontemporal_load(reinterpret_cast<const v4i32 *>(
                    a.wq + tile_src(lane, h, n0 + t * ROWS, a.N - 1, a.K, line_of(i) * LINE)));
    // the scales of the tile, requested behind the operands instead of cold at the end
    if (threadIdx.x < T * ROWS) ws_tile[threadIdx.x] = a.ws[min(n0 + (int)threadIdx.x, a.N - 1)];
    else if (threadIdx.x < T * ROWS + MAX_CHUNKS * ROWS)
        xs_tile[threadIdx.x - T * ROWS] = a.xs[min((int)threadIdx.x - T * ROWS, a.M - 1)];
    for (int o = threadIdx.x; o < chunks * T * 256; o += WAVES * 64) (&sums[0][0][0])[o] = 0;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            tile_park(patch, lane, wr[t][i][0], wr[t][i][1]);
            wr[t][i][0] = tile_take(patch, lane, kq);
            wr[t][i][1] = tile_take(patch, lane, 4 + kq);
        }
#pragma unroll 1
    for (int c = 0; c < chunks; ++c) {
        v4i32 acc[T];
#pragma unroll
        for (int t = 0; t < T; ++t) acc[t] = v4i32{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            tile_park(patch, lane, xr[i][0], xr[i][1]);
            const v4i32 x0 = tile_take(patch, lane, kq), x1 = tile_take(patch, lane, 4 + kq);
            if (wave + i * WAVES < lines) {  // uniform per wavefront
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, wr[t][i][0], acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, wr[t][i][1], acc[t], 0, 0, 0);
                }
            }
            if (c + 1 < chunks) request_x(c + 1, i);
        }
#pragma unroll
        for (int t = 0; t < T; ++t) {
            int32_t *dst = &sums[c * T + t][lane][0];
            atomicAdd(dst + 0, acc[t].x);
            atomicAdd(dst + 1, acc[t].y);
            atomicAdd(dst + 2, acc[t].z);
            atomicAdd(dst + 3, acc[t].w);
        }
    }
    __syncthreads();

    for (int o = threadIdx.x; o < chunks * T * 256; o += WAVES * 64) {
        const int ct = o >> 8, c = ct / T, t = ct % T, l = (o >> 2) & 63, v = o & 3;
        const int nl = t * ROWS + (l & 15), m = c * ROWS + 4 * (l >> 4) + v;
        const int n = n0 + nl;
        if (n < a.N && m < a.M) {
            const int sm = sums[ct][l][v];
            if (a.acc_out) a.acc_out[(size_t)m * a.N + n] = sm;
            a.y[(size_t)m * a.ldy + n] = (uint16_t)f32_to_bf16_bits(((float)sm * xs_tile[m]) * ws_tile[nl]);
        }
    }
}

template <int NLP, int WAVES, int T>
int launch128(const Args &a, hipStream_t st) {
    const dim3 grid((a.N + ROWS * T - 1) / (ROWS * T));
    gemm_w8a8_rows128_kernel<NLP, WAVES, T><<<grid, dim3(WAVES * 64), 0, st>>>(a);
    return check_launch("cmi_gemm_w8a8");
}

}  // namespace

namespace cmi {

// Two tiles per workgroup halve the activation bytes that go through L2 per chunk; measured faster
// (by 10-25 %) exactly where the halved grid still covers most of the CUs in a single round.
int gemm_w8a8_rows_tiles(int N) {
    const int wgs2 = (N + 2 * ROWS - 1) / (2 * ROWS);
    return wgs2 >= 160 && wgs2 <= 256 ? 2 : 1;
}

// Returns CMI_E_UNSUPPORTED without setting the error text when the shape is
// outside this kernel's range (the caller then uses a tiled kernel).
int gemm_w8a8_rows16(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws, void *y,
                     int32_t *acc_out, int M, int N, int K, int ldy, void *stream) {
    if (M < 1 || M > MAX_CHUNKS * ROWS || N < 1 || K < LINE || K % LINE != 0 || K > 80 * LINE)
        return CMI_E_UNSUPPORTED;
    if (!aligned(xq, 16) || !aligned(wq, 16)) return CMI_E_UNSUPPORTED;
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
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int lines = K / LINE;
    // eight wavefronts (shorter chains of dependent steps) measured 0.3-0.7 us faster up to
    // N = 19456; no difference at N = 151936
    const bool eight = (N + ROWS - 1) / ROWS <= 2048;
    if (M > ROWS) {
        const bool two = gemm_w8a8_rows_tiles(N) == 2;
        if (lines <= 8) return two ? launch128<2, 4, 2>(a, st) : launch128<2, 4, 1>(a, st);
        if (lines <= 24 && eight) return two ? launch128<3, 8, 2>(a, st) : launch128<3, 8, 1>(a, st);
        if (lines <= 20) return two ? launch128<5, 4, 2>(a, st) : launch128<5, 4, 1>(a, st);
        if (lines <= 40) return two ? launch128<5, 8, 2>(a, st) : launch128<5, 8, 1>(a, st);
        return two ? launch128<10, 8, 2>(a, st) : launch128<10, 8, 1>(a, st);
    }
    if (lines <= 8) return launch<2, 4>(a, st);
    if (lines <= 24 && eight) return launch<3, 8>(a, st);
    if (lines <= 20) return launch<5, 4>(a, st);
    if (lines <= 40) return launch<5, 8>(a, st);
    return launch<10, 8>(a, st);
}

}  // namespace cmi
