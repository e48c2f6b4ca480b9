// int8 weight-only GEMV for batches of up to 16 bf16 activation rows (batched
// decode, speculative verify).
//
//   y[m,n] = bf16( (sum_k x[m,k] * (float)wq[n,k]) * ws[n] )        fp32 sums
//
// With one row the kernel is a stream of weight bytes and a few dot-product
// instructions per 16 of them; with 16 rows the dot products alone (8 per row
// and 16 weight bytes) run at a quarter of memory speed.  int8 -> bf16 is exact
// and bf16 x bf16 products are exact in fp32, so here v_mfma_f32_16x16x32_bf16
// forms the sums -- 16 weight rows x 16 activation rows x 32 k per instruction
// -- and the vector ALU only widens the weight bytes.  The kernel stays a GEMV
// in every other respect: the weight is read once, straight into registers, all
// of a wavefront's bytes requested before anything else.
//
// A workgroup owns 16 weight rows; its wavefronts split K by 128-byte lines of
// the weight rows (wavefront w takes lines w, w+WAVES, ..).  For the MFMA lane l
// holds k  32*(l/16) .. +31  of a line for weight row l%16 (two 16-byte pieces)
// and for activation row l%16 (four pieces); both are fetched as whole cache
// lines and rearranged through private LDS patches.  The fp32 partial tiles of
// the wavefronts are added in wavefront order through LDS, so a row's result
// depends on K only, not on the batch it came in -- but it is not the bit
// pattern of the dot-product kernel behind cmi_gemv_w8a16 (different fp32
// summation order), which is why this kernel has an entry point of its own:
// callers that owe their users "a batched row equals the single-row call"
// (static-batch decode) stay on cmi_gemv_w8a16.
#include "rows16_tile.hpp"

namespace {

using namespace cmi;
using namespace cmi::rows16;

typedef float v4f32 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int ROWS = 16;
constexpr int LINE = 128;           // k per line
constexpr int XPITCH = 256 + 16;    // activation patch: 16 rows x 256 bytes
constexpr int XPATCH_BYTES = 16 * XPITCH;

struct Args {
    const int8_t *wq;
    const float *ws;
    const uint16_t *x;
    uint16_t *y;
    int M, N, K;
};

// Four int8 of a dword -> four bf16 (two dwords); exact.
__device__ __forceinline__ void widen4(uint32_t w, uint32_t &lo, uint32_t &hi) {
    const float f0 = (float)(int8_t)(w);
    const float f1 = (float)(int8_t)(w >> 8);
    const float f2 = (float)(int8_t)(w >> 16);
    const float f3 = (float)(int8_t)(w >> 24);
    // integers up to 128 in magnitude live in the upper 16 bits of their fp32 pattern
    lo = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
    hi = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
}

// NLP: lines per wavefront and round.  WAVES: wavefronts per workgroup.  ROUNDS: 1, or 2 for
// K above 128*NLP*WAVES (the second round's bytes are requested line by line as the first
// round frees their registers; asking for all weight bytes at the start took 179 registers
// and measured slower), or 0: as many rounds as K takes, counted at run time (K above 10240).
// T: 16-row tiles of weight rows per workgroup (the activation tiles a wavefront fetched and
// rearranged serve all of them: at 16 rows they are two thirds of the bytes a wavefront asks for).
template <int NLP, int WAVES, int ROUNDS, int T = 1>
__global__ void __launch_bounds__(WAVES * 64)
gemv_w8a16_rows16_kernel(const Args a) {
    static_assert(T == 1 || ROUNDS == 1, "several tiles only in the single-round arrangement");
    extern __shared__ __align__(16) uint8_t lds[];
    float(*partial)[64][4] = reinterpret_cast<float(*)[64][4]>(lds);  // [T * WAVES][64][4]
    uint8_t *patches = lds + T * WAVES * 1024;                            // per wavefront: weights, activations

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = lane >> 4;
    const int n0 = blockIdx.x * (T * ROWS);
    const int lines = a.K / LINE;
    uint8_t *wpatch = patches + wave * (PATCH_BYTES + XPATCH_BYTES), *xpatch = wpatch + PATCH_BYTES;
    const uint8_t *xbytes = reinterpret_cast<const uint8_t *>(a.x);
    auto line_of = [&](int r, int i) { return (r * NLP + i) * WAVES + wave; };

    // Activations first (L2 resident; memory answers in request order), then every weight byte.
    // An activation line is 256 bytes: parts 0 and 1, each fetched as two half tiles; rows past
    // M repeat the last one, their sums are dropped.
    v4i32 xr[NLP][4], wr[T][NLP][2];
    // One or two activation rows: every lane's row is one of two, so the MFMA arrangement (row
    // lane%16, bytes 64*kq .. +63 of the line) can be loaded as it is -- the requests collapse
    // onto a few cache lines -- and the LDS rearrangement is skipped.
    const bool direct_x = a.M <= 2;
    const uint8_t *xdirect = xbytes + (size_t)min(lane & 15, a.M - 1) * a.K * 2 + kq * 64;
    auto request_x = [&](int r, int i) {
        const int line = line_of(r, i);
        if (line >= lines) return;  // uniform per wavefront
        if (direct_x) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                xr[i][q] = *reinterpret_cast<const v4i32 *>(xdirect + line * 256 + q * 16);
            return;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q)
            xr[i][q] = *reinterpret_cast<const v4i32 *>(
                xbytes + tile_src(lane, q & 1, 0, a.M - 1, (size_t)a.K * 2, line * 256 + (q >> 1) * 128));
    };
    auto request_w = [&](int r, int i) {
        const int line = line_of(r, i);
        if (line >= lines) return;
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                wr[t][i][h] = __builtin_nontemporal_load(reinterpret_cast<const v4i32 *>(
                    a.wq + tile_src(lane, h, n0 + t * ROWS, a.N - 1, a.K, line * LINE)));
    };
#pragma unroll
    for (int i = 0; i < NLP; ++i) request_x(0, i);
#pragma unroll
    for (int i = 0; i < NLP; ++i) request_w(0, i);
    // The row scale of the output this thread will finish, requested now, behind everything the
    // arithmetic waits for: asked for at the end it is a cold load under a saturated memory system
    // (1.4 us of every workgroup's 4.6 us, by in-kernel timestamps).
    float ws_out[T];
#pragma unroll
    for (int t = 0; t < T; ++t) ws_out[t] = a.ws[min(n0 + t * ROWS + (int)((threadIdx.x >> 2) & 15), a.N - 1)];

    // the accumulator of lane l holds (n = l%16, m = 4*kq + v), v = 0..3, per tile
    v4f32 acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = v4f32{0.f, 0.f, 0.f, 0.f};
    const int rounds = ROUNDS > 0 ? ROUNDS : (lines + NLP * WAVES - 1) / (NLP * WAVES);
    constexpr int UNROLL = ROUNDS > 0 ? ROUNDS : 1;
#pragma unroll UNROLL
    for (int r = 0; r < rounds; ++r) {
        // activations into the MFMA arrangement: row lane%16, bytes 64*kq .. +63 of the line
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            if (direct_x || line_of(r, i) >= lines) break;
            uint8_t *p = xpatch + (lane >> 3) * XPITCH + (lane & 7) * 16;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *reinterpret_cast<v4i32 *>(p + (q & 1) * 8 * XPITCH + (q >> 1) * 128) = xr[i][q];
            const uint8_t *t = xpatch + (lane & 15) * XPITCH + kq * 64;
#pragma unroll
            for (int q = 0; q < 4; ++q) xr[i][q] = *reinterpret_cast<const v4i32 *>(t + q * 16);
        }
        // weights: rearrange, widen, multiply
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            if (line_of(r, i) >= lines) break;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                tile_park(wpatch, lane, wr[t][i][0], wr[t][i][1]);
                const v4i32 w0 = tile_take(wpatch, lane, 2 * kq), w1 = tile_take(wpatch, lane, 2 * kq + 1);
                const uint32_t d[8] = {(uint32_t)w0.x, (uint32_t)w0.y, (uint32_t)w0.z, (uint32_t)w0.w,
                                       (uint32_t)w1.x, (uint32_t)w1.y, (uint32_t)w1.z, (uint32_t)w1.w};
#pragma unroll
                for (int s = 0; s < 4; ++s) {  // k = 32*kq + 8*s .. +7 of the line
                    uint32_t b[4];
                    widen4(d[2 * s], b[0], b[1]);
                    widen4(d[2 * s + 1], b[2], b[3]);
                    const v4i32 bw = {(int)b[0], (int)b[1], (int)b[2], (int)b[3]};
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xr[i][s]),
                                                                     __builtin_bit_cast(bf16x8, bw), acc[t], 0, 0, 0);
                }
            }
            if (r + 1 < rounds) {
                request_x(r + 1, i);
                request_w(r + 1, i);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < T; ++t) *reinterpret_cast<v4f32 *>(&partial[t * WAVES + wave][lane][0]) = acc[t];
    __syncthreads();

    if (threadIdx.x < 256) {
        const int l = threadIdx.x >> 2, v = threadIdx.x & 3;
        const int m = 4 * (l >> 4) + v;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const int n = n0 + t * ROWS + (l & 15);
            if (n < a.N && m < a.M) {
                float total = partial[t * WAVES][l][v];
#pragma unroll
                for (int wv = 1; wv < WAVES; ++wv) total += partial[t * WAVES + wv][l][v];
                a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(total * ws_out[t]);
            }
        }
    }
}

template <int NLP, int WAVES, int ROUNDS = 1, int T = 1>
int launch(const Args &a, hipStream_t st) {
    constexpr int LDS_BYTES = WAVES * (T * 1024 + PATCH_BYTES + XPATCH_BYTES);
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemv_w8a16_rows16_kernel<NLP, WAVES, ROUNDS, T>),
                                   LDS_BYTES, devices, "cmi_gemv_w8a16_mfma"))
        return rc;
    const dim3 grid((a.N + T * ROWS - 1) / (T * ROWS));
    gemv_w8a16_rows16_kernel<NLP, WAVES, ROUNDS, T><<<grid, dim3(WAVES * 64), LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemv_w8a16_mfma");
}


// 17..64 activation rows: the workgroup still asks for its 16 weight rows once and keeps them in
// registers in the MFMA arrangement (NLP*ROUNDS lines per wavefront); the activation rows go
// through in chunks of 16, each with the arithmetic of the kernel above -- so a row's bits are
// the same as in a 16-row call -- and only the activations (L2 resident) and the widening are
// paid again per chunk.  The activation registers hold NLP lines: with two rounds a chunk is two
// such batches, and the batch after the one in hand is requested line by line as its registers
// free up.  The partial tiles of all chunks meet in LDS behind one barrier.
constexpr int MAX_CHUNKS = 4;

// T: 16-row tiles of weight rows per workgroup (single-round arrangements only): every workgroup
// pulls all activation rows through L2 once per chunk, M * K * 2 bytes times N / (16 T) workgroups,
// which from three chunks up is what the launch waits for.
template <int NLP, int WAVES, int ROUNDS, int T = 1>
__global__ void __launch_bounds__(WAVES * 64)
gemv_w8a16_rows64_kernel(const Args a) {
    static_assert(T == 1 || ROUNDS == 1, "several tiles only in the single-round arrangement");
    extern __shared__ __align__(16) uint8_t lds[];
    float(*partial)[64][4] = reinterpret_cast<float(*)[64][4]>(lds);  // [(chunk * T + tile) * WAVES + wave][64][4]
    const int chunks = (a.M + ROWS - 1) / ROWS;
    uint8_t *patches = lds + chunks * T * WAVES * 1024;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = lane >> 4;
    const int n0 = blockIdx.x * (T * ROWS);
    const int lines = a.K / LINE;
    uint8_t *wpatch = patches + wave * (PATCH_BYTES + XPATCH_BYTES), *xpatch = wpatch + PATCH_BYTES;
    const uint8_t *xbytes = reinterpret_cast<const uint8_t *>(a.x);
    auto line_of = [&](int r, int i) { return (r * NLP + i) * WAVES + wave; };

    v4i32 xr[NLP][4], wr[T][ROUNDS * NLP][2];
    auto request_x = [&](int c, int r, int i) {
        const int line = min(line_of(r, i), lines - 1);  // a slot past the last line is not used
#pragma unroll
        for (int q = 0; q < 4; ++q)
            xr[i][q] = *reinterpret_cast<const v4i32 *>(
                xbytes + tile_src(lane, q & 1, c * ROWS, a.M - 1, (size_t)a.K * 2, line * 256 + (q >> 1) * 128));
    };
#pragma unroll
    for (int i = 0; i < NLP; ++i) request_x(0, 0, i);
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r)
#pragma unroll
            for (int i = 0; i < NLP; ++i) {
                const int line = min(line_of(r, i), lines - 1);
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    wr[t][r * NLP + i][h] = __builtin_nontemporal_load(reinterpret_cast<const v4i32 *>(
                        a.wq + tile_src(lane, h, n0 + t * ROWS, a.N - 1, a.K, line * LINE)));
            }
    // the row scales of the outputs this thread will finish (n depends on the thread and the tile only),
    // requested behind the operands instead of cold at the end
    float ws_out[T];
#pragma unroll
    for (int t = 0; t < T; ++t) ws_out[t] = a.ws[min(n0 + t * ROWS + (int)((threadIdx.x >> 2) & 15), a.N - 1)];
    // weights into the MFMA arrangement, once
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int i = 0; i < ROUNDS * NLP; ++i) {
            tile_park(wpatch, lane, wr[t][i][0], wr[t][i][1]);
            wr[t][i][0] = tile_take(wpatch, lane, 2 * kq);
            wr[t][i][1] = tile_take(wpatch, lane, 2 * kq + 1);
        }

#pragma unroll 1
    for (int c = 0; c < chunks; ++c) {
        v4f32 acc[T];
#pragma unroll
        for (int t = 0; t < T; ++t) acc[t] = v4f32{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            // this batch of activation lines into the MFMA arrangement: row lane%16, bytes 64*kq .. +63
#pragma unroll
            for (int i = 0; i < NLP; ++i) {
                uint8_t *p = xpatch + (lane >> 3) * XPITCH + (lane & 7) * 16;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<v4i32 *>(p + (q & 1) * 8 * XPITCH + (q >> 1) * 128) = xr[i][q];
                const uint8_t *t = xpatch + (lane & 15) * XPITCH + kq * 64;
#pragma unroll
                for (int q = 0; q < 4; ++q) xr[i][q] = *reinterpret_cast<const v4i32 *>(t + q * 16);
            }
#pragma unroll
            for (int i = 0; i < NLP; ++i) {
                if (line_of(r, i) < lines) {  // uniform per wavefront
#pragma unroll
                    for (int t = 0; t < T; ++t) {
                        v4i32 w0 = wr[t][r * NLP + i][0], w1 = wr[t][r * NLP + i][1];
                        // with two rounds or several tiles of weight registers the widened copies must
                        // not be kept across chunks (the compiler would hoist them out of the loop and spill)
                        if (ROUNDS > 1 || T > 1) asm volatile("" : "+v"(w0), "+v"(w1));
                        const uint32_t d[8] = {(uint32_t)w0.x, (uint32_t)w0.y, (uint32_t)w0.z, (uint32_t)w0.w,
                                               (uint32_t)w1.x, (uint32_t)w1.y, (uint32_t)w1.z, (uint32_t)w1.w};
#pragma unroll
                        for (int s = 0; s < 4; ++s) {
                            uint32_t b[4];
                            widen4(d[2 * s], b[0], b[1]);
                            widen4(d[2 * s + 1], b[2], b[3]);
                            const v4i32 bw = {(int)b[0], (int)b[1], (int)b[2], (int)b[3]};
                            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xr[i][s]),
                                                                             __builtin_bit_cast(bf16x8, bw), acc[t], 0, 0, 0);
                        }
                    }
                }
                // this line's activation registers are free: ask for the same slot of the next batch
                if (r + 1 < ROUNDS) request_x(c, r + 1, i);
                else if (c + 1 < chunks) request_x(c + 1, 0, i);
            }
        }
#pragma unroll
        for (int t = 0; t < T; ++t) *reinterpret_cast<v4f32 *>(&partial[(c * T + t) * WAVES + wave][lane][0]) = acc[t];
    }
    __syncthreads();

    for (int o = threadIdx.x; o < chunks * T * 256; o += WAVES * 64) {
        const int ct = o >> 8, c = ct / T, t = ct % T, l = (o >> 2) & 63, v = o & 3;
        const int n = n0 + t * ROWS + (l & 15), m = c * ROWS + 4 * (l >> 4) + v;
        if (n < a.N && m < a.M) {
            float total = partial[ct * WAVES][l][v];
#pragma unroll
            for (int wv = 1; wv < WAVES; ++wv) total += partial[ct * WAVES + wv][l][v];
            float scale = ws_out[0];
#pragma unroll
            for (int tt = 1; tt < T; ++tt) scale = t == tt ? ws_out[tt] : scale;
            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(total * scale);
        }
    }
}

template <int NLP, int WAVES, int ROUNDS = 1, int T = 1>
int launch64(const Args &a, hipStream_t st) {
    constexpr int LDS_MAX = MAX_CHUNKS * T * WAVES * 1024 + WAVES * (PATCH_BYTES + XPATCH_BYTES);
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemv_w8a16_rows64_kernel<NLP, WAVES, ROUNDS, T>),
                                   LDS_MAX, devices, "cmi_gemv_w8a16_mfma"))
        return rc;
    const int chunks = (a.M + ROWS - 1) / ROWS;
    const int lds_bytes = chunks * T * WAVES * 1024 + WAVES * (PATCH_BYTES + XPATCH_BYTES);
    const dim3 grid((a.N + T * ROWS - 1) / (T * ROWS));
    gemv_w8a16_rows64_kernel<NLP, WAVES, ROUNDS, T><<<grid, dim3(WAVES * 64), lds_bytes, st>>>(a);
    return check_launch("cmi_gemv_w8a16_mfma");
}

}  // namespace

extern "C" int cmi_gemv_w8a16_mfma(const int8_t *wq, const float *ws, const void *x, void *y, int M, int N,
                                   int K, void *stream) {
    CMI_REQUIRE(wq && ws && x && y, CMI_E_ARG, "cmi_gemv_w8a16_mfma: null pointer");
    CMI_REQUIRE(M >= 1 && M <= MAX_CHUNKS * ROWS, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16_mfma: M=%d outside 1..64", M);
    CMI_REQUIRE(N >= 1 && K >= 1, CMI_E_ARG, "cmi_gemv_w8a16_mfma: bad shape N=%d K=%d", N, K);
    CMI_REQUIRE(K % LINE == 0, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16_mfma: K=%d is not a multiple of 128 (use cmi_gemv_w8a16)", K);
    CMI_REQUIRE(aligned(wq, 16) && aligned(x, 16) && aligned(y, 2) && aligned(ws, 4), CMI_E_ARG,
                "cmi_gemv_w8a16_mfma: wq and x must be 16-byte aligned");
    Args a;
    a.wq = wq;
    a.ws = ws;
    a.x = static_cast<const uint16_t *>(x);
    a.y = static_cast<uint16_t *>(y);
    a.M = M;
    a.N = N;
    a.K = K;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int lines = K / LINE;
    if (lines > 80) {
        // rows longer than two rounds of registers hold: the 16-row kernel with a round count read at
        // run time, 16 activation rows per launch (a row's bits are those of a 16-row call, as in the
        // 64-row kernel; the weight is read once per 16 rows)
        for (int lo = 0; lo < M; lo += ROWS) {
            Args part = a;
            part.x = a.x + (size_t)lo * K;
            part.y = a.y + (size_t)lo * N;
            part.M = M - lo < ROWS ? M - lo : ROWS;
            if (const int rc = launch<5, 8, 0>(part, st)) return rc;
        }
        return CMI_OK;
    }
    if (M > ROWS) {
        if (lines <= 8) return launch64<2, 4>(a, st);
        if (lines <= 20 && (N + ROWS - 1) / ROWS > 2048) return launch64<5, 4>(a, st);
        // Several weight tiles per workgroup: the activation rows a workgroup pulls through L2 per
        // chunk then serve 32 or 48 weight rows.  A launch takes (rounds of 256 workgroups) x (time of
        // a workgroup), and a workgroup of T tiles about (2 T + 1) units -- fitted to 2560 -> 9728 /
        // 6144 / 19456 and 4096 -> 11008 / 14336 / 5120 at 32..64 rows, where the best T follows this
        // count every time (64 rows of 2560 -> 9728: 21.9 -> 16.6 us with three tiles, 2560 -> 6144
        // 15.2 -> 12.6 with two, 4096 -> 14336 44 -> 39 with two; three is what LDS holds).
        const int tiles = (N + ROWS - 1) / ROWS;
        int T = 1, best = 1 << 30;
        for (int t = 1; t <= 3; ++t) {
            const int cost = ((tiles + t - 1) / t + 255) / 256 * (2 * t + 1);
            if (cost < best) best = cost, T = t;
        }
        if (lines <= 24) return T == 3 ? launch64<3, 8, 1, 3>(a, st) : T == 2 ? launch64<3, 8, 1, 2>(a, st) : launch64<3, 8>(a, st);
        if (lines <= 40) return T == 3 ? launch64<5, 8, 1, 3>(a, st) : T == 2 ? launch64<5, 8, 1, 2>(a, st) : launch64<5, 8>(a, st);
        return launch64<5, 8, 2>(a, st);
    }
    // eight wavefronts (shorter chains of dependent steps) up to 2048 workgroups, four beyond
    // (2560 -> 151936: 72 us against 84)
    // From four rows and 300 tiles of weight rows up, a workgroup owns two tiles: the activation
    // tiles its wavefronts fetched and rearranged serve both (16 rows: 2560 -> 6144 6.9 -> 6.3 us,
    // 2560 -> 151936 86 -> 78 us; with fewer rows or tiles one tile per workgroup stays faster).
    const int tiles = (N + ROWS - 1) / ROWS;
    const bool two = M >= 4 && tiles >= 300;
    if (lines <= 8) return launch<2, 4>(a, st);
    if (lines <= 20 && tiles > 2048) return two ? launch<5, 4, 1, 2>(a, st) : launch<5, 4>(a, st);
    if (lines <= 24) return two ? launch<3, 8, 1, 2>(a, st) : launch<3, 8>(a, st);
    if (lines <= 40) return two ? launch<5, 8, 1, 2>(a, st) : launch<5, 8>(a, st);
    return launch<5, 8, 2>(a, st);
}
