// W4A8 GEMV for up to 16 activation rows (speculative verify, small batches, long rows), from
// already quantised activations (K <= 10240 in one pass, longer rows in passes) or, up to 4
// rows and K <= 10240, from bf16 activations.
//
//   sum_g   = sum_{k in group g} xq[m,k] * (code(n,k) - 8)     int32, exact
//   total   = fma((float)sum_g, ws[n,g], total)                 g = 0,1,.. from 0.f
//   y[m,n]  = bf16(total * xs[m])
//
// HBM-bound on the packed weight, and meant to stay so: with 16 rows the
// v_dot4_i32_i8 formulation costs ~240 vector instructions per 16 weight bytes
// of a lane and runs at a quarter of memory speed.  The integer group sums are
// exact in any order, so they are formed by v_mfma_i32_16x16x64_i8 instead --
// 16 weight rows x 16 activation rows x 64 k per instruction -- which leaves the
// vector ALU only the nibble split and the fp32 chain.
//
// A workgroup owns 16 weight rows; its wavefronts split K by 128-byte lines of
// the weight rows (two groups of 128 k each), wavefront w taking lines w,
// w+WAVES, ..  (Two 16-row tiles per workgroup, sharing the activation
// registers, measured no faster.)  For the MFMA lane l holds weight row l%16 and
// the 32 k  128*g + 32*(l/16) ..  of a group: 16 packed bytes, whose low nibbles
// are k 8i..8i+3 and high nibbles k 8i+4..8i+7 of dword i.  The matching
// activation bytes are dwords 0,2,4,6 and 1,3,5,7 of the 32 contiguous xq bytes
// of row l%16, so both operands are plain 16-byte pieces.  They are fetched as
// whole cache lines and rearranged through a private LDS patch.  Codes stay
// unsigned; the -8 is applied by two more MFMAs against a constant operand of
// -8s (the matrix pipe is idle here).  Each wavefront parks its int32 group sums
// in LDS and, after one barrier, thread (n, m) walks the groups in ascending
// order.
#include "quant_math.hpp"
#include "rows16_tile.hpp"

namespace {

using namespace cmi;
using namespace cmi::rows16;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GS = 128;
constexpr int ROWS = 16;        // weight rows per workgroup = activation rows per MFMA
constexpr int MAX_K = 10240;    // 40 lines: 8 wavefronts x 5

constexpr int FUSED_ROWS = 4;   // rows the kernel quantises itself (bf16 activations in)
constexpr int FUSED_XV = 3;     // 16-byte bf16 vectors per thread and row: K <= 3 * 8 * threads

struct Args {
    const uint8_t *w4;
    const float *ws;
    const int8_t *xq;     // quantised activations and their scales, or
    const float *xs;
    const uint16_t *x;    // bf16 activations (FUSED), with optional copies of what was quantised
    int8_t *xq_out;
    float *xs_out;
    uint16_t *y;
    int32_t *group_acc;
    int M, N, K, G;
};

// group sums [G][64 lanes][4], scales [16][G], one rearrangement patch per wavefront; FUSED adds
// the int8 rows [4][K], their scales and the per-wavefront maxima
__host__ __device__ inline int lds_bytes(int G, int waves, bool fused = false) {
    return G * 1024 + ROWS * G * 4 + waves * PATCH_BYTES + (fused ? FUSED_ROWS * G * GS + 256 : 0);
}

// NLP: lines per wavefront.  WAVES: wavefronts per workgroup (4 or 8).
// DUMP: also write the int32 group sums to a.group_acc.
// FUSED: activations arrive as bf16 (up to 4 rows) and every workgroup quantises them itself
//        with the arithmetic of cmi_quant_act_i8 while its weights travel.
template <int NLP, int WAVES, bool DUMP, bool FUSED>
__global__ void __launch_bounds__(WAVES * 64)
gemv_w4a8_rows16_kernel(const Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    int32_t *sums = reinterpret_cast<int32_t *>(lds);             // [G][64 lanes][4]
    float *ws_lds = reinterpret_cast<float *>(lds + a.G * 1024);  // [16][G]

    uint8_t *patches = lds + a.G * 1024 + ROWS * a.G * 4;
    int8_t *xq_lds = reinterpret_cast<int8_t *>(patches + WAVES * PATCH_BYTES);             // FUSED: [4][K]
    float *xs_lds = reinterpret_cast<float *>(patches + WAVES * PATCH_BYTES + FUSED_ROWS * a.K);  // [4]
    float *part = xs_lds + 8;                                                                // [4][WAVES]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = lane >> 4;
    const int n0 = blockIdx.x * ROWS;
    const int lines = (a.G + 1) / 2;
    uint8_t *patch = patches + wave * PATCH_BYTES;

    // 1. activations of this wavefront's groups (L2 resident; asked for first because
    //    memory answers in request order); rows past M repeat the last one, their sums are dropped
    v4i32 xa[NLP][2][2];
    uint4 xv[FUSED ? FUSED_ROWS : 1][FUSED ? FUSED_XV : 1];
    const int xvecs = a.K / 8;
    if constexpr (FUSED) {
#pragma unroll
        for (int m = 0; m < FUSED_ROWS; ++m) {
            if (m >= a.M) break;  // uniform
            const uint4 *xg = reinterpret_cast<const uint4 *>(a.x + (size_t)m * a.K);
#pragma unroll
            for (int j = 0; j < FUSED_XV; ++j) {
                const int idx = threadIdx.x + j * (WAVES * 64);
                xv[m][j] = idx < xvecs ? xg[idx] : make_uint4(0, 0, 0, 0);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            const int line = wave + i * WAVES;
            if (line >= lines) break;  // uniform per wavefront
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int g = min(2 * line + h, a.G - 1);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    xa[i][h][j] =
                        *reinterpret_cast<const v4i32 *>(a.xq + tile_src(lane, j, 0, a.M - 1, a.K, g * GS));
            }
        }
    }
    // the activation scale of the output this thread will finish (m depends on the thread only),
    // requested now instead of cold at the end
    float xs_out = 0.f;
    if constexpr (!FUSED) xs_out = a.xs[min((int)(4 * ((threadIdx.x >> 6) & 3) + (threadIdx.x & 3)), a.M - 1)];
    // 2. the scales of the 16 rows (contiguous), into registers until the weights are asked for
    const int ws_total = min(ROWS, a.N - n0) * a.G;
    constexpr int WSN = (ROWS * (MAX_K / GS) + WAVES * 64 - 1) / (WAVES * 64);
    float wsreg[WSN];
    {
        const float *src = a.ws + (size_t)n0 * a.G;
#pragma unroll
        for (int i = 0; i < WSN; ++i) {
            const int idx = threadIdx.x + i * (WAVES * 64);
            wsreg[i] = idx < ws_total ? src[idx] : 0.f;
        }
    }
    // 3. every weight byte of this wavefront
    v4i32 w[NLP][2];
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
        const int line = wave + i * WAVES;
        if (line >= lines) break;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            w[i][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i32 *>(
                a.w4 + tile_src<true>(lane, j, n0, a.N - 1, a.K / 2, line * 128)));
    }
#pragma unroll
    for (int i = 0; i < WSN; ++i) {
        const int idx = threadIdx.x + i * (WAVES * 64);
        if (idx < ws_total) ws_lds[idx] = wsreg[i];
    }

    // 4. activations into the MFMA arrangement: row lane%16, bytes 32*kq .. +31 of each group
    if constexpr (FUSED) {
        // quantise the rows into LDS first (same bits as cmi_quant_act_i8), then read the pieces
#pragma unroll
        for (int m = 0; m < FUSED_ROWS; ++m) {
            if (m >= a.M) break;  // uniform
            float amax = 0.f;
#pragma unroll
            for (int j = 0; j < FUSED_XV; ++j)
                if (j * (WAVES * 64) < xvecs) amax = absmax8(xv[m][j], amax);  // uniform
            amax = wave_max_to_lane63(amax);
            if (lane == 63) part[m * WAVES + wave] = amax;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < FUSED_ROWS; ++m) {
            if (m >= a.M) break;  // uniform
            float amax = part[m * WAVES];
#pragma unroll
            for (int wv = 1; wv < WAVES; ++wv) amax = fmaxf(amax, part[m * WAVES + wv]);
            const RowScale rs = row_scale(amax);
            if (threadIdx.x == 0) {
                xs_lds[m] = rs.sc;
                if (a.xs_out && blockIdx.x == 0) a.xs_out[m] = rs.sc;
            }
#pragma unroll
            for (int j = 0; j < FUSED_XV; ++j) {
                const int idx = threadIdx.x + j * (WAVES * 64);
                if (j * (WAVES * 64) >= xvecs) break;  // uniform
                const uint2 q = quant8(xv[m][j], rs);
                if (idx < xvecs) {
                    reinterpret_cast<uint2 *>(xq_lds + (size_t)m * a.K)[idx] = q;
                    if (a.xq_out && blockIdx.x == 0)
                        reinterpret_cast<uint2 *>(a.xq_out + (size_t)m * a.K)[idx] = q;
                }
            }
        }
        __syncthreads();
        const int8_t *xrow = xq_lds + (size_t)min(lane & 15, min(a.M, FUSED_ROWS) - 1) * a.K + kq * 32;
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            const int line = wave + i * WAVES;
            if (line >= lines) break;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int g = min(2 * line + h, a.G - 1);
                xa[i][h][0] = *reinterpret_cast<const v4i32 *>(xrow + g * GS);
                xa[i][h][1] = *reinterpret_cast<const v4i32 *>(xrow + g * GS + 16);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            const int line = wave + i * WAVES;
            if (line >= lines) break;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                tile_park(patch, lane, xa[i][h][0], xa[i][h][1]);
                xa[i][h][0] = tile_take(patch, lane, 2 * kq);
                xa[i][h][1] = tile_take(patch, lane, 2 * kq + 1);
            }
        }
    }
    // 5. integer group sums: lane holds (n = lane%16, m = 4*kq + v), v = 0..3
    const v4i32 minus8 = {(int)0xF8F8F8F8u, (int)0xF8F8F8F8u, (int)0xF8F8F8F8u, (int)0xF8F8F8F8u};
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
        const int line = wave + i * WAVES;
        if (line >= lines) break;
        tile_park(patch, lane, w[i][0], w[i][1]);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int g = 2 * line + h;
            if (g >= a.G) break;  // uniform per wavefront
            const u32x4 ww = __builtin_bit_cast(u32x4, tile_take(patch, lane, 4 * h + kq));
            const v4i32 x0 = {xa[i][h][0].x, xa[i][h][0].z, xa[i][h][1].x, xa[i][h][1].z};
            const v4i32 x1 = {xa[i][h][0].y, xa[i][h][0].w, xa[i][h][1].y, xa[i][h][1].w};
            const u32x4 lo = ww & 0x0F0F0F0Fu, hi = (ww >> 4) & 0x0F0F0F0Fu;
            v4i32 acc = {0, 0, 0, 0};
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, minus8, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, minus8, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, __builtin_bit_cast(v4i32, lo), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, __builtin_bit_cast(v4i32, hi), acc, 0, 0, 0);
            reinterpret_cast<v4i32 *>(sums)[g * 64 + lane] = acc;
        }
    }
    __syncthreads();

    // 6. fp32 chain over the groups, one thread per (n, m)
    if (threadIdx.x < 256) {
        const int p = threadIdx.x;
        const int l = p >> 2, v = p & 3;
        const int nn = l & 15, m = 4 * (l >> 4) + v;
        const int n = n0 + nn;
        if (n < a.N && m < a.M) {
            const int32_t *sp = sums + p;
            const float *wsn = ws_lds + nn * a.G;
            float total = 0.f;
            int g = 0;
            for (; g + 4 <= a.G; g += 4) {
                int sv[4];
                float wv[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sv[i] = sp[(g + i) * 256];
                    wv[i] = wsn[g + i];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if constexpr (DUMP) a.group_acc[((size_t)m * a.G + g + i) * a.N + n] = sv[i];
                    total = fmaf((float)sv[i], wv[i], total);
                }
            }
            for (; g < a.G; ++g) {
                const int sg = sp[g * 256];
                if constexpr (DUMP) a.group_acc[((size_t)m * a.G + g) * a.N + n] = sg;
                total = fmaf((float)sg, wsn[g], total);
            }
            const float xsm = FUSED ? xs_lds[m] : xs_out;
            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(total * xsm);
        }
    }
}

template <int NLP, int WAVES, bool DUMP, bool FUSED>
int launch_one(const Args &a, hipStream_t st) {
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemv_w4a8_rows16_kernel<NLP, WAVES, DUMP, FUSED>),
                                   lds_bytes(MAX_K / GS, WAVES, FUSED), devices, "cmi_gemv_w4a8"))
        return rc;
    const dim3 grid((a.N + ROWS - 1) / ROWS);
    gemv_w4a8_rows16_kernel<NLP, WAVES, DUMP, FUSED>
        <<<grid, dim3(WAVES * 64), lds_bytes(a.G, WAVES, FUSED), st>>>(a);
    return check_launch("cmi_gemv_w4a8");
}

template <int NLP, int WAVES>
int launch(const Args &a, hipStream_t st) {
    if (a.x) {
        if (a.K > FUSED_XV * 8 * WAVES * 64) return CMI_E_UNSUPPORTED;
        return a.group_acc ? launch_one<NLP, WAVES, true, true>(a, st) : launch_one<NLP, WAVES, false, true>(a, st);
    }
    return a.group_acc ? launch_one<NLP, WAVES, true, false>(a, st) : launch_one<NLP, WAVES, false, false>(a, st);
}


// Rows longer than MAX_K: the same work in passes of 80 groups (10240 k), the fp32 chain carried
// from pass to pass in the register of its thread.  The next pass's bytes are requested as soon
// as this pass's MFMAs have consumed their registers, so memory keeps working while the chain of
// this pass runs.  Quantised activations only (a caller with bf16 rows quantises first).
constexpr int LONG_NLP = 3, LONG_WAVES = 8, LONG_GP = 2 * LONG_NLP * LONG_WAVES;  // groups per pass
constexpr int LONG_THREADS = LONG_WAVES * 64;
constexpr int LONG_WSN = (ROWS * LONG_GP + LONG_THREADS - 1) / LONG_THREADS;

template <bool DUMP>
__global__ void __launch_bounds__(LONG_THREADS)
gemv_w4a8_rows16_long_kernel(const Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    int32_t *sums = reinterpret_cast<int32_t *>(lds);                 // [LONG_GP][64 lanes][4]
    float *ws_lds = reinterpret_cast<float *>(lds + LONG_GP * 1024);  // [16][LONG_GP]
    uint8_t *patches = lds + LONG_GP * 1024 + ROWS * LONG_GP * 4;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = lane >> 4;
    const int n0 = blockIdx.x * ROWS;
    const int lines = (a.G + 1) / 2;
    const int passes = (a.G + LONG_GP - 1) / LONG_GP;
    const int nrows = min(ROWS, a.N - n0);
    uint8_t *patch = patches + wave * PATCH_BYTES;

    v4i32 xa[LONG_NLP][2][2], w[LONG_NLP][2];
    float wsreg[LONG_WSN];
    // requests of one pass: activations first, then the scales, then every weight byte
    auto request = [&](int pass) {
        const int line0 = pass * (LONG_NLP * LONG_WAVES) + wave;
#pragma unroll
        for (int i = 0; i < LONG_NLP; ++i) {
            const int line = line0 + i * LONG_WAVES;
            if (line >= lines) break;  // uniform per wavefront
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int g = min(2 * line + h, a.G - 1);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    xa[i][h][j] =
                        *reinterpret_cast<const v4i32 *>(a.xq + tile_src(lane, j, 0, a.M - 1, a.K, g * GS));
            }
        }
        const int gp = min(LONG_GP, a.G - pass * LONG_GP);  // groups of this pass
#pragma unroll
        for (int i = 0; i < LONG_WSN; ++i) {
            const int idx = threadIdx.x + i * LONG_THREADS;
            const int row = idx / LONG_GP, col = idx - row * LONG_GP;
            wsreg[i] = (row < nrows && col < gp) ? a.ws[(size_t)(n0 + row) * a.G + pass * LONG_GP + col] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < LONG_NLP; ++i) {
            const int line = line0 + i * LONG_WAVES;
            if (line >= lines) break;
#pragma unroll
            for (int j = 0; j < 2; ++j)
                w[i][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i32 *>(
                    a.w4 + tile_src<true>(lane, j, n0, a.N - 1, a.K / 2, line * 128)));
        }
    };
    request(0);

    const int p = threadIdx.x, l = (p >> 2) & 63, v = p & 3;
    const int nn = l & 15, m = 4 * (l >> 4) + v, n = n0 + nn;
    const bool chain = p < 256 && n < a.N && m < a.M;
    float total = 0.f;
    const v4i32 minus8 = {(int)0xF8F8F8F8u, (int)0xF8F8F8F8u, (int)0xF8F8F8F8u, (int)0xF8F8F8F8u};
#pragma unroll 1
    for (int pass = 0; pass < passes; ++pass) {
        const int line0 = pass * (LONG_NLP * LONG_WAVES) + wave;
        // scales of this pass (the previous pass's chain is behind the barrier that ended it)
#pragma unroll
        for (int i = 0; i < LONG_WSN; ++i) {
            const int idx = threadIdx.x + i * LONG_THREADS;
            if (idx < ROWS * LONG_GP) ws_lds[idx] = wsreg[i];
        }
        // activations into the MFMA arrangement: row lane%16, bytes 32*kq .. +31 of each group
#pragma unroll
        for (int i = 0; i < LONG_NLP; ++i) {
            if (line0 + i * LONG_WAVES >= lines) break;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                tile_park(patch, lane, xa[i][h][0], xa[i][h][1]);
                xa[i][h][0] = tile_take(patch, lane, 2 * kq);
                xa[i][h][1] = tile_take(patch, lane, 2 * kq + 1);
            }
        }
        // integer group sums: lane holds (n = lane%16, m = 4*kq + v), v = 0..3
#pragma unroll
        for (int i = 0; i < LONG_NLP; ++i) {
            const int line = line0 + i * LONG_WAVES;
            if (line >= lines) break;
            tile_park(patch, lane, w[i][0], w[i][1]);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int g = 2 * line + h;
                if (g >= a.G) break;  // uniform per wavefront
                const u32x4 ww = __builtin_bit_cast(u32x4, tile_take(patch, lane, 4 * h + kq));
                const v4i32 x0 = {xa[i][h][0].x, xa[i][h][0].z, xa[i][h][1].x, xa[i][h][1].z};
                const v4i32 x1 = {xa[i][h][0].y, xa[i][h][0].w, xa[i][h][1].y, xa[i][h][1].w};
                const u32x4 lo = ww & 0x0F0F0F0Fu, hi = (ww >> 4) & 0x0F0F0F0Fu;
                v4i32 acc = {0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, minus8, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, minus8, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, __builtin_bit_cast(v4i32, lo), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, __builtin_bit_cast(v4i32, hi), acc, 0, 0, 0);
                reinterpret_cast<v4i32 *>(sums)[(g - pass * LONG_GP) * 64 + lane] = acc;
            }
        }
        if (pass + 1 < passes) request(pass + 1);
        __syncthreads();
        // fp32 chain over this pass's groups, one thread per (n, m)
        if (chain) {
            const int gp = min(LONG_GP, a.G - pass * LONG_GP);
            const int32_t *sp = sums + p;
            const float *wsn = ws_lds + nn * LONG_GP;
            int g = 0;
            for (; g + 4 <= gp; g += 4) {
                int sv[4];
                float wv[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sv[i] = sp[(g + i) * 256];
                    wv[i] = wsn[g + i];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if constexpr (DUMP) a.group_acc[((size_t)m * a.G + pass * LONG_GP + g + i) * a.N + n] = sv[i];
                    total = fmaf((float)sv[i], wv[i], total);
                }
            }
            for (; g < gp; ++g) {
                const int sg = sp[g * 256];
                if constexpr (DUMP) a.group_acc[((size_t)m * a.G + pass * LONG_GP + g) * a.N + n] = sg;
                total = fmaf((float)sg, wsn[g], total);
            }
        }
        __syncthreads();  // sums and scales are overwritten by the next pass
    }
    if (chain) a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(total * a.xs[m]);
}

template <bool DUMP>
int launch_long(const Args &a, hipStream_t st) {
    constexpr int LDS_BYTES = LONG_GP * 1024 + ROWS * LONG_GP * 4 + LONG_WAVES * PATCH_BYTES;
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemv_w4a8_rows16_long_kernel<DUMP>), LDS_BYTES,
                                   devices, "cmi_gemv_w4a8"))
        return rc;
    const dim3 grid((a.N + ROWS - 1) / ROWS);
    gemv_w4a8_rows16_long_kernel<DUMP><<<grid, dim3(LONG_THREADS), LDS_BYTES, st>>>(a);
    return check_launch("cmi_gemv_w4a8");
}


// 17..128 quantised activation rows, K <= 10240: the workgroup's 16 weight rows are asked for once
// and stay in registers as the MFMA pieces; the activation rows go through in chunks of 16, each
// with the group sums, the barrier and the fp32 chain of the 16-row kernel (so the bits are the
// same), the next chunk's activations requested as soon as this chunk's MFMAs have consumed their
// registers.
constexpr int MAX_CHUNKS = 8;

template <int NLP, int WAVES, bool DUMP>
__global__ void __launch_bounds__(WAVES * 64)
gemv_w4a8_rows128_kernel(const Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    int32_t *sums = reinterpret_cast<int32_t *>(lds);             // [G][64 lanes][4]
    float *ws_lds = reinterpret_cast<float *>(lds + a.G * 1024);  // [16][G]
    uint8_t *patches = lds + a.G * 1024 + ROWS * a.G * 4;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = lane >> 4;
    const int n0 = blockIdx.x * ROWS;
    const int lines = (a.G + 1) / 2;
    const int chunks = (a.M + ROWS - 1) / ROWS;
    uint8_t *patch = patches + wave * PATCH_BYTES;

    v4i32 xa[NLP][2][2], w[NLP][2];
    auto request_x = [&](int c) {
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            const int line = wave + i * WAVES;
            if (line >= lines) break;  // uniform per wavefront
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int g = min(2 * line + h, a.G - 1);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    xa[i][h][j] = *reinterpret_cast<const v4i32 *>(
                        a.xq + tile_src(lane, j, c * ROWS, a.M - 1, a.K, g * GS));
            }
        }
    };
    request_x(0);
    const int ws_total = min(ROWS, a.N - n0) * a.G;
    constexpr int WSN = (ROWS * (MAX_K / GS) + WAVES * 64 - 1) / (WAVES * 64);
    float wsreg[WSN];
    {
        const float *src = a.ws + (size_t)n0 * a.G;
#pragma unroll
        for (int i = 0; i < WSN; ++i) {
            const int idx = threadIdx.x + i * (WAVES * 64);
            wsreg[i] = idx < ws_total ? src[idx] : 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
        const int line = wave + i * WAVES;
        if (line >= lines) break;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            w[i][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i32 *>(
                a.w4 + tile_src<true>(lane, j, n0, a.N - 1, a.K / 2, line * 128)));
    }
#pragma unroll
    for (int i = 0; i < WSN; ++i) {
        const int idx = threadIdx.x + i * (WAVES * 64);
        if (idx < ws_total) ws_lds[idx] = wsreg[i];
    }
    // weights into the MFMA pieces, once: piece 4*h + kq of the line for group 2*line + h
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
        if (wave + i * WAVES >= lines) break;
        tile_park(patch, lane, w[i][0], w[i][1]);
        w[i][0] = tile_take(patch, lane, kq);
        w[i][1] = tile_take(patch, lane, 4 + kq);
    }

    const int p = threadIdx.x, l = (p >> 2) & 63, v = p & 3;
    const int nn = l & 15, n = n0 + nn;
    const v4i32 minus8 = {(int)0xF8F8F8F8u, (int)0xF8F8F8F8u, (int)0xF8F8F8F8u, (int)0xF8F8F8F8u};
#pragma unroll 1
    for (int c = 0; c < chunks; ++c) {
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            if (wave + i * WAVES >= lines) break;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                tile_park(patch, lane, xa[i][h][0], xa[i][h][1]);
                xa[i][h][0] = tile_take(patch, lane, 2 * kq);
                xa[i][h][1] = tile_take(patch, lane, 2 * kq + 1);
            }
        }
#pragma unroll
        for (int i = 0; i < NLP; ++i) {
            const int line = wave + i * WAVES;
            if (line >= lines) break;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int g = 2 * line + h;
                if (g >= a.G) break;  // uniform per wavefront
                const u32x4 ww = __builtin_bit_cast(u32x4, w[i][h]);
                const v4i32 x0 = {xa[i][h][0].x, xa[i][h][0].z, xa[i][h][1].x, xa[i][h][1].z};
                const v4i32 x1 = {xa[i][h][0].y, xa[i][h][0].w, xa[i][h][1].y, xa[i][h][1].w};
                const u32x4 lo = ww & 0x0F0F0F0Fu, hi = (ww >> 4) & 0x0F0F0F0Fu;
                v4i32 acc = {0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, minus8, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, minus8, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, __builtin_bit_cast(v4i32, lo), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, __builtin_bit_cast(v4i32, hi), acc, 0, 0, 0);
                reinterpret_cast<v4i32 *>(sums)[g * 64 + lane] = acc;
            }
        }
        if (c + 1 < chunks) request_x(c + 1);
        __syncthreads();
        const int m = c * ROWS + 4 * (l >> 4) + v;
        if (p < 256 && n < a.N && m < a.M) {
            const int32_t *sp = sums + p;
            const float *wsn = ws_lds + nn * a.G;
            float total = 0.f;
            int g = 0;
            for (; g + 4 <= a.G; g += 4) {
                int sv[4];
                float wv[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sv[i] = sp[(g + i) * 256];
                    wv[i] = wsn[g + i];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if constexpr (DUMP) a.group_acc[((size_t)m * a.G + g + i) * a.N + n] = sv[i];
                    total = fmaf((float)sv[i], wv[i], total);
                }
            }
            for (; g < a.G; ++g) {
                const int sg = sp[g * 256];
                if constexpr (DUMP) a.group_acc[((size_t)m * a.G + g) * a.N + n] = sg;
                total = fmaf((float)sg, wsn[g], total);
            }
            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(total * a.xs[m]);
        }
        __syncthreads();  // the next chunk overwrites the sums
    }
}

template <int NLP, int WAVES>
int launch128(const Args &a, hipStream_t st) {
    static std::atomic<uint64_t> devices{0};
    const void *fn = a.group_acc ? reinterpret_cast<const void *>(gemv_w4a8_rows128_kernel<NLP, WAVES, true>)
                                 : reinterpret_cast<const void *>(gemv_w4a8_rows128_kernel<NLP, WAVES, false>);
    static std::atomic<uint64_t> devices_dump{0};
    if (const int rc = reserve_lds(fn, lds_bytes(MAX_K / GS, WAVES), a.group_acc ? devices_dump : devices, "cmi_gemv_w4a8"))
        return rc;
    const dim3 grid((a.N + ROWS - 1) / ROWS);
    if (a.group_acc)
        gemv_w4a8_rows128_kernel<NLP, WAVES, true><<<grid, dim3(WAVES * 64), lds_bytes(a.G, WAVES), st>>>(a);
    else
        gemv_w4a8_rows128_kernel<NLP, WAVES, false><<<grid, dim3(WAVES * 64), lds_bytes(a.G, WAVES), st>>>(a);
    return check_launch("cmi_gemv_w4a8");
}

}  // namespace

namespace cmi {

// Exactly one of xq/xs (quantised rows, up to 16) and x (bf16 rows, up to 4: the kernel quantises
// them itself and copies what it used to xq_out / xs_out when given) is set.  Returns
// CMI_E_UNSUPPORTED without setting the error text when the shape is outside this kernel's range
// (the caller then uses another kernel).
int gemv_w4a8_rows16(const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs, const void *x,
                     void *y, int32_t *group_acc, int8_t *xq_out, float *xs_out, int M, int N, int K,
                     void *stream) {
    if (M < 1 || M > (x ? FUSED_ROWS : MAX_CHUNKS * ROWS) || K < GS || K % GS != 0 || N < 1) return CMI_E_UNSUPPORTED;
    if (K > MAX_K && (x || M > ROWS)) return CMI_E_UNSUPPORTED;
    Args a;
    a.w4 = w4;
    a.ws = ws;
    a.xq = xq;
    a.xs = xs;
    a.x = static_cast<const uint16_t *>(x);
    a.xq_out = xq_out;
    a.xs_out = xs_out;
    a.y = static_cast<uint16_t *>(y);
    a.group_acc = group_acc;
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = K / GS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (K > MAX_K) return group_acc ? launch_long<true>(a, st) : launch_long<false>(a, st);
    const int lines = (a.G + 1) / 2;
    // Eight wavefronts per workgroup beyond 20 lines, and up to ~640 workgroups (2.5 per compute
    // unit) where a wavefront's chain of dependent steps is what is left to shorten (0.6-0.9 us
    // faster at N = 2560..9728); four on larger grids (7 % faster at N = 151936).
    const int grid = (N + ROWS - 1) / ROWS;
    const bool eight = lines > 20 || (grid <= 640 && lines >= 8);
    if (M > ROWS) {
        if (!eight) {
            switch ((lines + 3) / 4) {
                case 1: return launch128<1, 4>(a, st);
                case 2: return launch128<2, 4>(a, st);
                case 3: return launch128<3, 4>(a, st);
                case 4: return launch128<4, 4>(a, st);
                default: return launch128<5, 4>(a, st);
            }
        }
        switch ((lines + 7) / 8) {
            case 1: return launch128<1, 8>(a, st);
            case 2: return launch128<2, 8>(a, st);
            case 3: return launch128<3, 8>(a, st);
            case 4: return launch128<4, 8>(a, st);
            default: return launch128<5, 8>(a, st);
        }
    }
    if (!eight) {
        switch ((lines + 3) / 4) {
            case 1: return launch<1, 4>(a, st);
            case 2: return launch<2, 4>(a, st);
            case 3: return launch<3, 4>(a, st);
            case 4: return launch<4, 4>(a, st);
            default: return launch<5, 4>(a, st);
        }
    }
    switch ((lines + 7) / 8) {
        case 1: return launch<1, 8>(a, st);
        case 2: return launch<2, 8>(a, st);
        case 3: return launch<3, 8>(a, st);
        case 4: return launch<4, 8>(a, st);
        default: return launch<5, 8>(a, st);
    }
}

}  // namespace cmi
