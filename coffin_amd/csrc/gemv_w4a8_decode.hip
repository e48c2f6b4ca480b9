// W4A8 decode GEMV: bf16 activations in, 1..4 rows, K <= 10240, one launch.
//
//   xq, xs  = per-token int8 quantisation of x (arithmetic of cmi_quant_act_i8)
//   sum_g   = sum_{k in group g} xq[m,k] * (code(n,k) - 8)     int32, exact
//   total   = fma((float)sum_g, ws[n,g], total)                 g = 0,1,.. from 0.f
//   y[m,n]  = bf16(total * xs[m])
//
// HBM-bound on the packed weight (half a byte per element).  One wavefront owns
// four weight rows, a quarter-wavefront (16 lanes x 16 B = 256 B per load) each,
// and requests the whole of its rows before it does anything else, so memory
// sees every byte of the launch in flight from the first microsecond; a
// workgroup is four such wavefronts.  While the weights travel the workgroup
// quantises the activations into LDS (every workgroup redoes this small job:
// it saves a launch and the int8 round trip), together with -8 * sum(xq) per
// 32-element chunk -- the start value of the v_dot4_i32_i8 accumulators, which
// lets the unsigned codes be used without re-biasing -- and the per-group
// scales of its 16 rows.  Four adjacent lanes own one group of 128 k; their
// int32 partials are added with two DPP quad permutes and parked in LDS, where
// one lane per (row, m) walks the groups in order: the fp32 chain is order
// sensitive and must not depend on how K was spread over lanes.
#include "quant_math.hpp"

namespace {

using namespace cmi;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GS = 128;
constexpr int ROWS_PER_WAVE = 4;
constexpr int MAX_K = 10240;
// 16-byte bf16 vectors per thread and activation row so that a workgroup of WV wavefronts carries K <= MAX_K
constexpr int xv_of(int wv) { return (MAX_K / 8 + 64 * wv - 1) / (64 * wv); }

struct Args {
    const uint8_t *w4;
    const float *ws;
    const uint16_t *x;   // bf16 activations (PREQ == false)
    const int8_t *xq;    // quantised activations and their scales (PREQ == true)
    const float *xs;
    uint16_t *y;
    int32_t *group_acc;
    int8_t *xq_out;
    float *xs_out;
    int M, N, K, G;
};

// LDS carve-up (bytes); every part 16-byte aligned.
struct Lds {
    int xq, xsum, wsc, sums, xs, part, total;
};
// Weight rows of a workgroup of wv wavefronts: every wavefront four rows of its own, or (ksplit)
// every four wavefronts four shared rows.
__host__ __device__ constexpr int rows_per_block(int wv, bool ksplit) { return ROWS_PER_WAVE * (ksplit ? wv / 4 : wv); }

__host__ __device__ inline Lds lds_layout(int mt, int K, bool ksplit, int wv) {
    const int G = K / GS;
    const int rows = rows_per_block(wv, ksplit);
    Lds l;
    l.xq = 0;
    l.xsum = l.xq + mt * K;                           // int8 [mt][K]
    l.wsc = l.xsum + mt * (K / 32) * 4;               // int32 [mt][K/32]
    l.sums = l.wsc + ((rows * G * 4 + 15) & ~15);     // float [rows][G]
    l.xs = l.sums + rows * ((G + 3) & ~3) * mt * 4;   // int32 [rows][mt][G padded to 4]
    l.part = l.xs + 16 * 4;                           // float [mt] (padded to 16)
    l.total = l.part + 4 * wv * 4;                    // float [mt][wv], mt <= 4
    return l;
}

// M: activation-row tile (1, 2, 4).  NL: 256-byte loads per weight row and wavefront.
// KSPLIT: the four wavefronts of a workgroup share four weight rows and take every fourth
//         256-byte piece each (few, long rows: more workgroups, same bytes in flight);
//         otherwise each wavefront owns four rows of its own.
// PREQ:   activations arrive already quantised (a.xq, a.xs) instead of as bf16.
// WV:     wavefronts per workgroup, 4 or 16.  Every workgroup quantises the whole activation row for
//         itself; sixteen wavefronts do that once for four times as many weight rows.
template <int M, int NL, bool KSPLIT, bool PREQ, int WV>
__global__ void __launch_bounds__(64 * WV)
gemv_w4a8_decode_kernel(const Args a) {
    constexpr int THREADS = 64 * WV;
    extern __shared__ __align__(16) uint8_t lds[];
    const Lds L = lds_layout(M, a.K, KSPLIT, WV);
    int8_t *xq_lds = reinterpret_cast<int8_t *>(lds + L.xq);
    int32_t *xsum_lds = reinterpret_cast<int32_t *>(lds + L.xsum);
    float *ws_lds = reinterpret_cast<float *>(lds + L.wsc);
    int32_t *sums = reinterpret_cast<int32_t *>(lds + L.sums);
    float *xs_lds = reinterpret_cast<float *>(lds + L.xs);
    float *part = reinterpret_cast<float *>(lds + L.part);

    constexpr int RPB = rows_per_block(WV, KSPLIT);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q16 = lane & 15, r = lane >> 4;
    const int n0 = blockIdx.x * RPB;
    // first row of this wavefront inside the workgroup, and (ksplit) which quarter of each row it takes
    const int wrow0 = (KSPLIT ? (wave >> 2) : wave) * ROWS_PER_WAVE;
    const int kpart = wave & 3;
    const int nrow = min(n0 + wrow0 + r, a.N - 1);
    const int row_bytes = a.K / 2;
    const int nchunks = a.K / 32;

    // 1. activations first (memory answers in request order and they are needed first)
    constexpr int XVN = PREQ ? (xv_of(WV) + 1) / 2 : xv_of(WV);  // 16-byte vectors per thread and row
    const int xvecs = PREQ ? a.K / 16 : a.K / 8;
    uint4 v[M][XVN];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int mrow = m < a.M ? m : a.M - 1;
        const uint4 *xg = PREQ ? reinterpret_cast<const uint4 *>(a.xq + (size_t)mrow * a.K)
                               : reinterpret_cast<const uint4 *>(a.x + (size_t)mrow * a.K);
#pragma unroll
        for (int j = 0; j < XVN; ++j) {
            const int idx = threadIdx.x + j * THREADS;
            v[m][j] = idx < xvecs ? xg[idx] : make_uint4(0, 0, 0, 0);
        }
    }
    // 2. the per-group scales of the workgroup's rows (contiguous in memory), into registers
    // for now: they must not be waited for after the weights, which return in request order
    constexpr int WSV = (RPB * (MAX_K / GS) + THREADS - 1) / THREADS;  // floats per thread: RPB rows x G <= 80
    const int ws_total = min(RPB, a.N - n0) * a.G;
    float wsreg[WSV];
    {
        const float *src = a.ws + (size_t)n0 * a.G;
#pragma unroll
        for (int i = 0; i < WSV; ++i) {
            const int idx = threadIdx.x + i * THREADS;
            wsreg[i] = idx < ws_total ? src[idx] : 0.f;
        }
    }
    // 3. every weight byte this wavefront is responsible for
    const u32x4 *wrow = reinterpret_cast<const u32x4 *>(a.w4 + (size_t)nrow * row_bytes);
    auto chunk_of = [&](int j) { return (KSPLIT ? j * 4 + kpart : j) * 16 + q16; };  // 16-byte chunk = 32 k
    u32x4 w[NL];
#pragma unroll
    for (int j = 0; j < NL; ++j) w[j] = __builtin_nontemporal_load(wrow + min(chunk_of(j), nchunks - 1));
#pragma unroll
    for (int i = 0; i < WSV; ++i) {
        const int idx = threadIdx.x + i * THREADS;
        if (idx < ws_total) ws_lds[idx] = wsreg[i];
    }

    // 4. int8 rows, their scales and -8 * (sum of each 32-element chunk) into LDS
    if constexpr (PREQ) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            if (threadIdx.x == 0) xs_lds[m] = a.xs[m < a.M ? m : a.M - 1];
#pragma unroll
            for (int j = 0; j < XVN; ++j) {
                if (j * THREADS >= xvecs) break;  // uniform
                const int idx = threadIdx.x + j * THREADS;
                const uint4 q = v[m][j];
                int s8 = __builtin_amdgcn_sdot4((int)q.x, 0x01010101, 0, false);
                s8 = __builtin_amdgcn_sdot4((int)q.y, 0x01010101, s8, false);
                s8 = __builtin_amdgcn_sdot4((int)q.z, 0x01010101, s8, false);
                s8 = __builtin_amdgcn_sdot4((int)q.w, 0x01010101, s8, false);
                s8 += dpp_i32<0xB1, 0xf>(s8);  // two consecutive vectors = one chunk
                if (idx < xvecs) {
                    reinterpret_cast<uint4 *>(xq_lds + (size_t)m * a.K)[idx] = q;
                    if ((idx & 1) == 0) xsum_lds[m * nchunks + (idx >> 1)] = -8 * s8;
                }
            }
        }
    } else {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float amax = 0.f;
#pragma unroll
            for (int j = 0; j < XVN; ++j)
                if (j * THREADS < xvecs) amax = absmax8(v[m][j], amax);  // uniform: skip vectors past K
            amax = wave_max_to_lane63(amax);
            if (lane == 63) part[m * WV + wave] = amax;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float amax = part[m * WV];
#pragma unroll
            for (int w = 1; w < WV; ++w) amax = fmaxf(amax, part[m * WV + w]);
            const RowScale rs = row_scale(amax);
            const float sc = rs.sc;
            if (threadIdx.x == 0) {
                xs_lds[m] = sc;
                if (a.xs_out && blockIdx.x == 0 && m < a.M) a.xs_out[m] = sc;
            }
#pragma unroll
            for (int j = 0; j < XVN; ++j) {
                if (j * THREADS >= xvecs) break;  // uniform
                const int idx = threadIdx.x + j * THREADS;
                const uint2 q = quant8(v[m][j], rs);
                // four consecutive vectors (adjacent lanes) = one chunk
                int s8 = __builtin_amdgcn_sdot4((int)q.x, 0x01010101, 0, false);
                s8 = __builtin_amdgcn_sdot4((int)q.y, 0x01010101, s8, false);
                s8 += dpp_i32<0xB1, 0xf>(s8);  // quad_perm [1,0,3,2]
                s8 += dpp_i32<0x4E, 0xf>(s8);  // quad_perm [2,3,0,1]
                if (idx < xvecs) {
                    reinterpret_cast<uint2 *>(xq_lds + (size_t)m * a.K)[idx] = q;
                    if ((idx & 3) == 0) xsum_lds[m * nchunks + (idx >> 2)] = -8 * s8;
                    if (a.xq_out && blockIdx.x == 0 && m < a.M)
                        reinterpret_cast<uint2 *>(a.xq_out + (size_t)m * a.K)[idx] = q;
                }
            }
        }
    }
    __syncthreads();

    // 5. integer group sums
    // [row of the wavefront][m][group]: the lane that walks a row's groups reads them 16 bytes at a time
    const int Gpad = (a.G + 3) & ~3;
    int32_t *wsums = sums + (wrow0 / ROWS_PER_WAVE) * (Gpad * ROWS_PER_WAVE * M);
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        if ((KSPLIT ? j * 4 + kpart : j) * 16 >= nchunks) break;  // uniform per wavefront
        const int c = chunk_of(j);
        const bool live = c < nchunks;
        const int cs = live ? c : nchunks - 1;
        const uint32_t ww[4] = {w[j].x, w[j].y, w[j].z, w[j].w};
        uint32_t op[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            op[2 * i] = ww[i] & 0x0F0F0F0Fu;
            op[2 * i + 1] = (ww[i] >> 4) & 0x0F0F0F0Fu;
        }
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const uint4 *xp = reinterpret_cast<const uint4 *>(xq_lds + (size_t)m * a.K) + 2 * cs;
            const uint4 x0 = xp[0], x1 = xp[1];
            const uint32_t xv[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            int acc = xsum_lds[m * nchunks + cs];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = __builtin_amdgcn_sdot4((int)op[i], (int)xv[i], acc, false);
            acc += dpp_i32<0xB1, 0xf>(acc);
            acc += dpp_i32<0x4E, 0xf>(acc);
            if ((lane & 3) == 0 && live) wsums[(r * M + m) * Gpad + (c >> 2)] = acc;
        }
    }
    if constexpr (KSPLIT) {
        __syncthreads();
        if (kpart != 0) return;
    } else {
        // the group sums below were written by this wavefront itself
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
    }

    // 6. fp32 chain over the groups, one lane per (row, m).  The integer sums go out first, all
    // lanes sharing the work, so that the chain itself is free of branches and stores.
    if (a.group_acc) {
        const int n_out = ROWS_PER_WAVE * M * a.G;
        for (int i = lane; i < n_out; i += 64) {
            const int rm = i / a.G, g = i - rm * a.G;
            const int rr = rm / M, m = rm - rr * M;
            const int n = n0 + wrow0 + rr;
            if (n < a.N && m < a.M) a.group_acc[((size_t)m * a.G + g) * a.N + n] = wsums[rm * Gpad + g];
        }
    }
    if (lane < ROWS_PER_WAVE * M) {
        const int rr = lane / M, m = lane - rr * M;
        const int brow = wrow0 + rr;  // row within the workgroup
        const int n = n0 + brow;
        if (n < a.N && m < a.M) {
            const float *wsn = ws_lds + brow * a.G;
            const int32_t *sn = wsums + (rr * M + m) * Gpad;
            float total = 0.f;
            int g = 0;
            if ((a.G & 3) == 0) {
                // Eight groups per trip, read as 16-byte vectors with the next trip's reads in
                // flight during this trip's chain (one convert and one fma per group, each fma
                // waiting for the last).
                const v4i32 *sv = reinterpret_cast<const v4i32 *>(sn);
                const float4 *wv = reinterpret_cast<const float4 *>(wsn);
                auto chain4 = [&](const v4i32 &sq, const float4 &wq) {
                    total = fmaf((float)sq[0], wq.x, total);
                    total = fmaf((float)sq[1], wq.y, total);
                    total = fmaf((float)sq[2], wq.z, total);
                    total = fmaf((float)sq[3], wq.w, total);
                };
                const int quads = a.G >> 2;
                int q = 0;
                if (quads >= 2) {
                    v4i32 s0 = sv[0], s1 = sv[1];
                    float4 w0 = wv[0], w1 = wv[1];
                    for (; q + 4 <= quads; q += 2) {
                        const v4i32 t0 = sv[q + 2], t1 = sv[q + 3];
                        const float4 u0 = wv[q + 2], u1 = wv[q + 3];
                        chain4(s0, w0);
                        chain4(s1, w1);
                        s0 = t0, s1 = t1, w0 = u0, w1 = u1;
                    }
                    chain4(s0, w0);
                    chain4(s1, w1);
                    q += 2;
                }
                if (q < quads) chain4(sv[q], wv[q]);
                g = a.G;
            }
            for (; g < a.G; ++g) total = fmaf((float)sn[g], wsn[g], total);
            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(total * xs_lds[m]);
        }
    }
}

template <int M, int NL, bool KSPLIT, bool PREQ, int WV>
int launch(const Args &a, hipStream_t st) {
    const Lds L = lds_layout(M, a.K, KSPLIT, WV);
    if (L.total > 64 * 1024) return CMI_E_UNSUPPORTED;
    constexpr int RPB = rows_per_block(WV, KSPLIT);
    const dim3 grid((a.N + RPB - 1) / RPB);
    gemv_w4a8_decode_kernel<M, NL, KSPLIT, PREQ, WV><<<grid, dim3(64 * WV), L.total, st>>>(a);
    return check_launch("cmi_gemv_w4a8");
}

template <int M, bool PREQ, int WV>
int dispatch_wv(const Args &a, hipStream_t st, bool ksplit) {
    const int pieces = (a.K + 511) / 512;  // 256-byte pieces per weight row
    if (ksplit) {
        const int nl = (pieces + 3) / 4;
        if (nl <= 2) return launch<M, 2, true, PREQ, WV>(a, st);
        if (nl <= 5) return launch<M, 5, true, PREQ, WV>(a, st);
        return CMI_E_UNSUPPORTED;
    }
    if (pieces <= 5) return launch<M, 5, false, PREQ, WV>(a, st);
    if (pieces <= 8) return launch<M, 8, false, PREQ, WV>(a, st);
    if (pieces <= 10) return launch<M, 10, false, PREQ, WV>(a, st);
    if (pieces <= 20) return launch<M, 20, false, PREQ, WV>(a, st);
    return CMI_E_UNSUPPORTED;
}

template <int M, bool PREQ>
int dispatch(const Args &a, hipStream_t st) {
    const int pieces = (a.K + 511) / 512;
    // few rows: share each row among four wavefronts so that the grid still covers the chip
    // (below one 16-row workgroup per compute unit; at 384 workgroups whole rows per wavefront are
    // faster: 2560 -> 6144 takes 5.1 us against 6.3)
    const bool ksplit = (a.N + 15) / 16 < 256 && pieces >= 4;
    // Quantising from bf16, every workgroup redoes the whole activation row: with sixteen
    // wavefronts a workgroup does it for four times the weight rows.  That pays where rows are
    // shared among wavefronts (few long rows, each workgroup quantising a long row for four
    // weight rows: 4096 -> 2560 4.8 -> 4.2 us, 9728 -> 2560 8.6 -> 8.2 us); with whole rows per
    // wavefront the wider barriers cost more than the quantisation saved (2560 -> 19456
    // 8.5 -> 9.9 us).  One bf16 row only (the decode case).
    const int opt = option_w4_decode_waves();
    const bool wide = opt ? opt == 16 : (!PREQ && M == 1 && ksplit);
    if constexpr (M == 1) {
        if (wide) return dispatch_wv<M, PREQ, 16>(a, st, ksplit);
    }
    return dispatch_wv<M, PREQ, 4>(a, st, ksplit);
}

// Variant of gemv_w4a8_chain for this shape (lanes per weight row + 100 * wavefronts per row +
// 10000 * wavefronts per workgroup), or 0 to stay with the kernel of this file.  Measured per
// projection, quantised rows / bf16 rows, against this file's kernel:
//   2560 -> 6144   3.6 / 4.0 us (4.3 / 4.7)      4096 -> 2560   3.2 / 3.6 us (3.6 / 4.1)
//   2560 -> 19456  6.2 / 7.3 us (7.1 / 8.3)      9728 -> 2560   5.6 / 7.5 us (5.9 / 8.1)
int chain_variant(int M, int N, int K, bool from_bf16) {
    const int opt = option_w4_decode_chain();
    if (opt == 1 || M > 2) return 0;
    if (opt) return opt;
    if (K <= 5120) {
        // sixteen lanes per row (four rows per wavefront); from bf16 rows, a grid of one to two
        // 16-row workgroups per compute unit is better served by 32-row workgroups (half as many
        // of them repeat the quantisation)
        const int wgs16 = (N + 15) / 16;
        return from_bf16 && wgs16 > 256 && wgs16 <= 512 ? 40108 : 40116;
    }
    // longer rows: four wavefronts (quantised rows) or two of an eight-wavefront workgroup (bf16
    // rows) share a row
    return from_bf16 ? 80216 : 40416;
}

}  // namespace

namespace cmi {

// Exactly one of x (bf16) and xq/xs (already quantised) is given.  Returns
// CMI_E_UNSUPPORTED without setting the error text when the shape is outside
// this kernel's range (the caller then uses the general kernel).
int gemv_w4a8_decode(const uint8_t *w4, const float *ws, const void *x, const int8_t *xq, const float *xs,
                     void *y, int32_t *group_acc, int8_t *xq_out, float *xs_out, int M, int N, int K,
                     void *stream) {
    if (M < 1 || M > 4 || K < GS || K % GS != 0 || N < 1) return CMI_E_UNSUPPORTED;
    // the chain-in-registers kernel where it applies (and is not switched off)
    if (const int variant = chain_variant(M, N, K, x != nullptr)) {
        const int rc = gemv_w4a8_chain(w4, ws, x, xq, xs, y, group_acc, xq_out, xs_out, M, N, K, variant, stream);
        if (rc != CMI_E_UNSUPPORTED) return rc;
    }
    if (K > MAX_K) return CMI_E_UNSUPPORTED;
    Args a;
    a.w4 = w4;
    a.ws = ws;
    a.x = static_cast<const uint16_t *>(x);
    a.xq = xq;
    a.xs = xs;
    a.y = static_cast<uint16_t *>(y);
    a.group_acc = group_acc;
    a.xq_out = xq_out;
    a.xs_out = xs_out;
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = K / GS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x) {
        if (M <= 1) return dispatch<1, false>(a, st);
        if (M <= 2) return dispatch<2, false>(a, st);
        return dispatch<4, false>(a, st);
    }
    if (M <= 1) return dispatch<1, true>(a, st);
    if (M <= 2) return dispatch<2, true>(a, st);
    return dispatch<4, true>(a, st);
}

}  // namespace cmi
