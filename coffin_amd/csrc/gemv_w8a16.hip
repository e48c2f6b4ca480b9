// int8 weight-only GEMV for 1..16 activation rows: y = bf16(ws[n] * sum_k wq[n,k] x[m,k]).
//
// HBM-bound: the only large stream is the int8 weight, read exactly once with
// 16-byte loads that are contiguous across the wavefront (1 KiB per
// wave-load).  No MFMA: int8 is widened in registers (SDWA convert + byte
// permute to packed bf16, exact for |w| <= 127) and multiplied against packed
// bf16 activations with v_dot2c_f32_bf16, fp32 accumulation.
//
// Canonical summation order (what makes a batched row bit-identical to the
// single-row call, whatever blocking the launcher picks); it depends on K only:
//   - K is cut into segments of 1024 (64 lanes x 16 elements); lane l of
//     segment s owns elements [s*1024 + l*16, +16);
//   - U consecutive segments form a unit (U = unit_segments(K), 1..4);
//   - inside a unit a lane accumulates its products in k order into one fp32
//     chain that starts at 0.f (eight chained dot2 per segment, segments
//     ascending);
//   - the 64 lane chains of a unit are summed by the fixed DPP tree
//     wave_sum_to_lane63;
//   - unit totals are added in ascending unit order, starting from unit 0's
//     total (not from 0.f);
//   - the per-row weight scale multiplies that sum once, then one bf16 rounding.
//
// Execution: one wavefront = (block of R weight rows, one unit of K).  All of a
// wavefront's weight loads are issued up front and there are many small
// wavefronts (R = 2: 2 KiB x CHT in flight each, ~70 VGPRs), which is what keeps
// HBM saturated from the first microsecond to the last: the hardware dispatcher
// back-fills retiring wavefronts, so late memory service of one wavefront never
// idles the rest.  The activations are the same few cache lines for every
// wavefront on the chip; fetched per wavefront they serialise on the L2
// channels that own those lines, so a workgroup (4 wavefronts, 16 for 16 rows)
// copies them into LDS once -- requested before the weights, because memory
// returns data in issue order -- and every wavefront reads its fragments from
// there, at most 4 activation rows in registers at a time (for 4 rows and more
// in an order that makes the reads free of bank conflicts).  Batches whose
// activations do not fit LDS are split into narrower calls.  A unit wider than
// the register budget of M rows is walked in sub-trips with the next sub-trip's
// weights in flight.  When K spans several units the wavefronts of a team each take units
// of the same rows and the unit totals meet in LDS (summed in unit order by one
// lane per output); otherwise lane 63, which holds the tree result, scales and
// stores.  From four activation rows on the 8..32 lane sums of a wavefront go through
// the tree together (wave_sum_transposed: same pairing, same bits, a lane keeping half
// of its values per level) and end in as many lanes, which store in parallel.  A single activation row against a K of two or three units (and against a
// mid-sized weight with K in one unit) takes gemv_w8a16_wholerow_kernel instead: one
// wavefront per weight row, all units.

#include "gemv_w8a16_math.hpp"

#include <cstdlib>

namespace {

using namespace cmi;

struct GemvArgs {
    const int8_t *wq;
    const float *ws;
    const uint16_t *x;
    uint16_t *y;
    int M, N, K;
    int nchunks;    // K / 16
    int nseg;       // ceil(nchunks / 64)
    int unit;       // segments per unit (canonical, from K)
    int units;      // ceil(nseg / unit)
    int subtrips;   // ceil(unit / CHT)
    uint32_t xvecs_rcp;  // ceil(2^32 / (K/8)): idx / (K/8) == umulhi(idx, xvecs_rcp) for idx < 2^16
    int nblocks;    // ceil(N / R)
    int uw;         // wavefronts of a team (they stride over the units)
    uint32_t uw_rcp;  // ceil(2^16 / uw)
    int teams;      // row blocks per workgroup
};

// Wavefronts per workgroup (they share one LDS copy of the activations); wide
// batches get smaller workgroups so that each wavefront may use more registers.
// (For one row and K in several units, 9728 -> 2560, that means one team of 3 wavefronts that
// stages the whole activation row for two weight rows; workgroups of 6, 9 and 12 wavefronts stage
// less and measured 8.6, 9.3 and 9.7 us against 7.3.)
// Four rows and more with K in several units (a team is then 3 or 4 wavefronts that share two
// weight rows): sixteen wavefronts, or every two weight rows would pay for staging the whole
// activation block (9728 -> 2560 at 4 rows: 19 us with 4 wavefronts, 16 with 8, 9 with 16).
constexpr int block_waves(int m, int mode = 0, bool multi_unit = false) {
    return m >= 16 ? 16 : (m >= 4 && multi_unit) ? 16 : m >= 8 ? 8 : (m == 4 && mode == 2) ? 8 : 4;
}
constexpr int max_block_waves(int m, int mode) { return (m >= 4 && mode != 0) ? 16 : block_waves(m); }

// Wavefronts per SIMD the register allocation must leave room for.
constexpr int simd_waves(int m, int cht) { return m >= 8 || (m == 4 && cht == 1) ? 4 : 1; }

// uint4 vectors of the LDS copy of the activations.
//   From 4 rows: [segment][row of the M tile][half][lane], 2 KiB per (segment, row), the tail of
//     the last segment and any dead segments zeroed: reads are contiguous across lanes, rows
//     differ by a compile-time offset and dead chunks read zeros without a select.
//   Up to 2 rows, K one unit: [row][segment][lane][half], i.e. a row as it is in memory, padded
//     with zeros to whole segments: again no select, a lane's address is its own offset plus
//     constants.
//   Up to 2 rows, several units: [row][K] unpadded plus one zeroed 32-byte slot that dead chunks
//     are pointed at (padding whole dead segments would cost a workgroup per CU at K = 9728).
__host__ __device__ constexpr int xlds_vectors(int mt, int rows, int K, int segs, bool one_unit) {
    return mt >= 4 ? mt * segs * 128 : one_unit ? rows * segs * 128 : rows * (K / 8) + 2;
}

// Activation rows held in registers at a time; wider batches loop over tiles of this many
// (4 rows = 32 registers: with accumulators and weights the kernel stays under 128, which
// 4 wavefronts per SIMD need; a spill inside the K loop costs a memory round trip each).
constexpr int m_tile(int m) { return m < 4 ? m : 4; }

// 16-byte vectors of activations each thread can carry from global memory to LDS, and the
// short variant that covers the decode shapes of up to four rows (e.g. K up to 4096 at four
// wavefronts and one row).
constexpr int xstage_vectors(int m) { return m <= 1 ? 8 : m <= 2 ? 16 : m <= 4 ? 20 : 8; }
constexpr int xstage_short(int m) { return m <= 1 ? 2 : m <= 2 ? 4 : m <= 4 ? 6 : xstage_vectors(m); }

template <int M, int CHT>
struct XStage {
    uint4 x[M][CHT][2];
};

template <int R, int CHT>
struct WStage {
    u32x4 w[R][CHT];
};

// MODE 0: K is one unit that fits one sub-trip (no loop, no unit exchange).
// MODE 1: several units, each one sub-trip (all loads up front, totals via LDS).
// MODE 2: general: units walked in pipelined sub-trips.
// XLDS: the workgroup stages the activations in LDS; otherwise each wavefront
//       reads them from global memory (only when they do not fit).
// XV: 16-byte vectors of activations each thread carries from global memory to LDS.
template <int M, int R, int CHT, int MODE, bool XLDS, int XV>
__global__ void __launch_bounds__(64 * max_block_waves(M, MODE), simd_waves(M, CHT))
gemv_w8a16_kernel(const GemvArgs a) {
    extern __shared__ uint4 smem[];  // staged activations (XLDS, see xlds_vectors), then unit totals
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: row addresses stay scalar
    // a single unit means one wavefront per team; otherwise wave / uw through a 16-bit reciprocal
    // (exact for the at most 16 wavefronts of a workgroup)
    const int team = MODE == 0 ? wave : (int)(((uint32_t)wave * a.uw_rcp) >> 16);
    const int rb = xcd_contiguous_block(blockIdx.x, gridDim.x) * a.teams + team;
    const bool idle = rb >= a.nblocks;  // only in the last workgroup
    int u = wave - team * a.uw;         // unit in hand; the team's wavefronts stride over units
    const int xvecs = a.K / 8;          // uint4 per activation row
    const int segs = a.units * a.unit;  // segments the unit loop walks (>= nseg)
    float *unit_total = reinterpret_cast<float *>(smem + (XLDS ? xlds_vectors(M, a.M, a.K, segs, MODE == 0) : 0)) +
                        team * a.units * (R * M);

    const int8_t *wrow[R];  // uniform per wavefront
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int n = rb * R + r;
        n = n < a.N ? n : a.N - 1;
        wrow[r] = a.wq + (size_t)n * a.K;
    }

    // Loads are unconditional: a dead chunk's address is clamped to the row's
    // last chunk and its activations are zeroed, so nothing branches between a
    // load and the arithmetic it overlaps.
    auto load_w = [&](WStage<R, CHT> &s, int unit_idx, int t) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < CHT; ++j) {
                const int chunk = (unit_idx * a.unit + t * CHT + j) * 64 + lane;
                s.w[r][j] = __builtin_nontemporal_load(
                    reinterpret_cast<const u32x4 *>(wrow[r] + (uint32_t)min(chunk, a.nchunks - 1) * 16u));
            }
    };
    constexpr int MT = m_tile(M), MH = M / MT;
    int xoff = 0;  // always 0; carries the ordering dependency described at its asm
    auto load_x = [&](XStage<MT, CHT> &s, int unit_idx, int t, int mh) {
        const int seg_end = min((unit_idx + 1) * a.unit, a.nseg);
#pragma unroll
        for (int j = 0; j < CHT; ++j) {
            const int seg = unit_idx * a.unit + t * CHT + j;
            const int chunk = seg * 64 + lane;
            const bool live = seg < seg_end && chunk < a.nchunks;
            const int safe = min(chunk, a.nchunks - 1);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int mrow = mh * MT + m < a.M ? mh * MT + m : a.M - 1;
                if constexpr (XLDS) {
                    // dead chunks read zeros: the LDS reads are unconditional
                    if constexpr (M >= 4) {
                        const int at = (seg * M + mh * MT + m) * 128 + lane + xoff;
                        s.x[m][j][0] = smem[at];
                        s.x[m][j][1] = smem[at + 64];
                    } else if constexpr (MODE == 0) {
                        const int at = (mrow * segs + seg) * 128 + 2 * lane;
                        s.x[m][j][0] = smem[at];
                        s.x[m][j][1] = smem[at + 1];
                    } else {
                        // a select on the address, so the LDS reads stay unconditional
                        const int at = live ? mrow * xvecs + 2 * chunk : a.M * xvecs;
                        s.x[m][j][0] = smem[at];
                        s.x[m][j][1] = smem[at + 1];
                    }
                } else {
                    const uint4 *xp = reinterpret_cast<const uint4 *>(a.x + (size_t)mrow * a.K);
                    const uint4 lo = xp[2 * safe], hi = xp[2 * safe + 1];
                    s.x[m][j][0] = live ? lo : make_uint4(0, 0, 0, 0);
                    s.x[m][j][1] = live ? hi : make_uint4(0, 0, 0, 0);
                }
            }
        }
    };

    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = 0.f;

    auto compute = [&](const WStage<R, CHT> &ws_, const XStage<MT, CHT> &xs_, int mh) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int j = 0; j < CHT; ++j) {
                bf16x2_t wb[8];
                widen4(ws_.w[r][j].x, wb[0], wb[1]);
                widen4(ws_.w[r][j].y, wb[2], wb[3]);
                widen4(ws_.w[r][j].z, wb[4], wb[5]);
                widen4(ws_.w[r][j].w, wb[6], wb[7]);
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const uint32_t xv[8] = {xs_.x[m][j][0].x, xs_.x[m][j][0].y, xs_.x[m][j][0].z,
                                            xs_.x[m][j][0].w, xs_.x[m][j][1].x, xs_.x[m][j][1].y,
                                            xs_.x[m][j][1].z, xs_.x[m][j][1].w};
                    float v = acc[r][mh * MT + m];
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        v = __builtin_amdgcn_fdot2_f32_bf16(wb[i], __builtin_bit_cast(bf16x2_t, xv[i]),
                                                            v, false);
                    acc[r][mh * MT + m] = v;
                }
            }
        }
    };

    // Activation fetch first (memory returns data in issue order, so whatever a
    // wavefront waits for must have been requested before the long weight
    // stream), then all first-trip weights, then the LDS hand-over: the copy and
    // its barrier run in the shadow of the weight latency.
    uint4 xstage[XV];
    const int xtotal = a.M * xvecs;
    if constexpr (XLDS) {
        const uint4 *xg = reinterpret_cast<const uint4 *>(a.x);
        // (the zero of the idle threads also keeps the compiler from moving a load down to the
        // predicated LDS store that consumes it, behind the weight requests)
#pragma unroll
        for (int j = 0; j < XV; ++j) {
            const int idx = threadIdx.x + j * blockDim.x;
            xstage[j] = idx < xtotal ? xg[idx] : make_uint4(0, 0, 0, 0);
        }
    }
    WStage<R, CHT> w0;
    load_w(w0, min(u, a.units - 1), 0);
    // Row scales: uniform per wavefront, but fetched as vector loads behind the weights (the
    // opaque zero keeps the address in a vector register).  As scalar loads they would share the
    // LDS counter and sit in front of the barrier of the activation hand-over.
    int vzero = 0;
    asm volatile("" : "+v"(vzero));
    float scale[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int n = rb * R + r;
        scale[r] = a.ws[(n < a.N ? n : a.N - 1) + vzero];
    }
    // several units: the lane that adds the unit totals of output (r, m) = (lane / M, lane % M)
    // scales it; its scale is requested here, not cold at the end
    float scale_fin = 0.f;
    if constexpr (MODE != 0) scale_fin = a.ws[min(rb * R + min(lane / M, R - 1), a.N - 1)];
    // Four rows and more: the R * M lane sums of a unit are reduced together (wave_sum_transposed:
    // the same tree, a sixth of the adds at 32 values) and the total of output (r, m) =
    // (tidx / M, tidx % M) ends in lane < R * M, which scales and stores it -- one store per
    // wavefront instead of R * M from lane 63.
    constexpr bool TRANSPOSED = R * M >= 8;
    int tidx = 0;
    float scale_lane = 0.f, tot = 0.f;
    if constexpr (TRANSPOSED) {
        tidx = wave_sum_transposed_index<R * M>(lane);
        if constexpr (MODE == 0) scale_lane = a.ws[min(rb * R + tidx / M, a.N - 1)];
    }
    if constexpr (XLDS) {
#pragma unroll
        for (int j = 0; j < XV; ++j) {
            const int idx = threadIdx.x + j * blockDim.x;
            // Within a segment (64 chunks of 16 weights) the first halves of all chunks
            // come first, then the second halves: a wavefront's 16-byte reads are then
            // contiguous across lanes (no bank conflicts).
            const bool mine = idx < xtotal;
            if constexpr (M >= 4) {
                const int row = __umulhi((uint32_t)idx, a.xvecs_rcp);
                const int v = idx - row * xvecs;
                const int seg = v >> 7, half = v & 1, c = (v & 127) >> 1;
                if (mine) smem[(seg * M + row) * 128 + half * 64 + c] = xstage[j];
            } else {
                // little LDS traffic: memory order; the second row starts at its padded offset
                const int row = idx >= xvecs ? 1 : 0;
                const int pad = MODE == 0 ? segs * 128 - xvecs : 0;
                if (mine) smem[idx + row * pad] = xstage[j];
            }
        }
        if constexpr (M >= 4) {
            // zero what no activation covers: lanes past K in the last segment, dead segments
            const int last = a.nseg - 1, cl = a.nchunks - last * 64;  // chunks in the last segment
            const int tail = 64 - cl;                                  // zero vectors per (row, half) there
            const int n_tail = a.M * 2 * tail;
            for (int i = threadIdx.x; i < n_tail; i += blockDim.x) {
                const int row = i / (2 * tail), rem = i - row * 2 * tail;
                const int half = rem / tail, c = cl + rem - half * tail;
                smem[(last * M + row) * 128 + half * 64 + c] = make_uint4(0, 0, 0, 0);
            }
            const int n_dead = (segs - a.nseg) * M * 128;
            for (int i = threadIdx.x; i < n_dead; i += blockDim.x)
                smem[a.nseg * M * 128 + i] = make_uint4(0, 0, 0, 0);
        } else if constexpr (MODE == 0) {
            const int pad = segs * 128 - xvecs;  // zero vectors behind each row (< 128)
            for (int i = threadIdx.x; i < a.M * pad; i += blockDim.x) {
                const int row = i >= pad ? 1 : 0;
                smem[row * segs * 128 + xvecs + i - row * pad] = make_uint4(0, 0, 0, 0);
            }
        } else {
            if (threadIdx.x < 2) smem[xtotal + threadIdx.x] = make_uint4(0, 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll 1
    for (; u < a.units; u += a.uw) {
        if (idle) break;
        XStage<MT, CHT> x0;
        auto consume = [&](const WStage<R, CHT> &w, int t) {
#pragma unroll
            for (int mh = 0; mh < MH; ++mh) {
                // keep one activation tile in registers: no LDS reads of the next
                // tile hoisted above this one's arithmetic (other wavefronts fill in)
                load_x(x0, u, t, mh);
                compute(w, x0, mh);
                // Wide batches: the next tile's LDS address is made to depend on this
                // tile's sums, so only one activation tile is ever live in registers
                // (other wavefronts of the SIMD cover the LDS latency).
                if constexpr (M >= 8) {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        float *p = &acc[r][mh * MT];
                        asm volatile("" : "+v"(p[0]), "+v"(p[1]), "+v"(p[2]), "+v"(p[3]), "+v"(xoff));
                    }
                }
            }
        };
        if constexpr (MODE != 2) {
            consume(w0, 0);
        } else {
            // sub-trips of the unit, next weights in flight while these are consumed
            WStage<R, CHT> w1;
            int t = 0;
#pragma unroll 1
            for (; t + 2 < a.subtrips; t += 2) {
                load_w(w1, u, t + 1);
                consume(w0, t);
                load_w(w0, u, t + 2);
                consume(w1, t + 1);
            }
            if (t + 1 < a.subtrips) {
                load_w(w1, u, t + 1);
                consume(w0, t);
                consume(w1, t + 1);
            } else {
                consume(w0, t);
            }
        }
        if (MODE != 0 && u + a.uw < a.units) load_w(w0, u + a.uw, 0);  // next unit of this wavefront
        if constexpr (TRANSPOSED) {
            float flat[R * M];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int m = 0; m < M; ++m) flat[r * M + m] = acc[r][m];
            tot = wave_sum_transposed<R * M>(flat, lane);
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int m = 0; m < M; ++m) acc[r][m] = wave_sum_to_lane63(acc[r][m]);
        }
        if constexpr (MODE == 0) break;
        // unit totals meet in LDS; one lane per output adds them in unit order below
        if constexpr (TRANSPOSED) {
            if (lane < R * M) unit_total[u * (R * M) + tidx] = tot;
        } else if (lane == 63) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int m = 0; m < M; ++m) unit_total[u * (R * M) + r * M + m] = acc[r][m];
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) acc[r][m] = 0.f;
    }

    if constexpr (MODE == 0 && TRANSPOSED) {
        const int r = tidx / M, m = tidx - r * M;
        const int n = rb * R + r;
        if (!idle && lane < R * M && n < a.N && m < a.M)
            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(scale_lane * tot);
    } else if constexpr (MODE == 0) {
        if (!idle && lane == 63) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int n = rb * R + r;
                if (n < a.N) {
#pragma unroll
                    for (int m = 0; m < M; ++m)
                        if (m < a.M)
                            a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(scale[r] * acc[r][m]);
                }
            }
        }
    } else {
        __syncthreads();
        if (!idle && wave == team * a.uw && lane < R * M) {
            const int r = lane / M, m = lane - r * M;
            const int n = rb * R + r;
            if (n < a.N && m < a.M) {
                float total = unit_total[lane];
                for (int v = 1; v < a.units; ++v) total += unit_total[v * (R * M) + lane];
                a.y[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(scale_fin * total);
            }
        }
    }
}

// One activation row, K in up to three units of one sub-trip each: a wavefront owns a whole
// weight row -- all units, every byte requested up front -- and adds its unit totals in lane
// 63 in the canonical order, so there is no exchange through LDS and no second barrier, and a
// workgroup of W wavefronts stages the activation row once for W weight rows (the team
// arrangement of the general kernel stages it once per two rows).  Same bits.
template <int CHT, int NU, int XV>
__global__ void __launch_bounds__(256)
gemv_w8a16_wholerow_kernel(const GemvArgs a) {
    extern __shared__ uint4 smem[];  // the activation row, then one zeroed 32-byte slot
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int n_raw = xcd_contiguous_block(blockIdx.x, gridDim.x) * waves + wave;
    const int n = n_raw < a.N ? n_raw : a.N - 1;
    const int8_t *wrow = a.wq + (size_t)n * a.K;
    const int xvecs = a.K / 8;

    uint4 xstage[XV];
    const uint4 *xg = reinterpret_cast<const uint4 *>(a.x);
#pragma unroll
    for (int j = 0; j < XV; ++j) {
        const int idx = threadIdx.x + j * blockDim.x;
        xstage[j] = idx < xvecs ? xg[idx] : make_uint4(0, 0, 0, 0);
    }
    u32x4 w[NU][CHT];
#pragma unroll
    for (int u = 0; u < NU; ++u)
#pragma unroll
        for (int j = 0; j < CHT; ++j) {
            const int chunk = ((u * CHT + j) * 64 + lane);
            w[u][j] = __builtin_nontemporal_load(
                reinterpret_cast<const u32x4 *>(wrow + (uint32_t)min(chunk, a.nchunks - 1) * 16u));
        }
    int vzero = 0;
    asm volatile("" : "+v"(vzero));
    const float scale = a.ws[n + vzero];
#pragma unroll
    for (int j = 0; j < XV; ++j) {
        const int idx = threadIdx.x + j * blockDim.x;
        if (idx < xvecs) smem[idx] = xstage[j];
    }
    if (threadIdx.x < 2) smem[xvecs + threadIdx.x] = make_uint4(0, 0, 0, 0);
    __syncthreads();

    float total = 0.f;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const int seg_end = min((u + 1) * CHT, a.nseg);
        float v = 0.f;
#pragma unroll
        for (int j = 0; j < CHT; ++j) {
            const int seg = u * CHT + j;
            const int chunk = seg * 64 + lane;
            const bool live = seg < seg_end && chunk < a.nchunks;
            const int at = live ? 2 * chunk : xvecs;
            const uint4 x0 = smem[at], x1 = smem[at + 1];
            bf16x2_t wb[8];
            widen4(w[u][j].x, wb[0], wb[1]);
            widen4(w[u][j].y, wb[2], wb[3]);
            widen4(w[u][j].z, wb[4], wb[5]);
            widen4(w[u][j].w, wb[6], wb[7]);
            const uint32_t xv[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i)
                v = __builtin_amdgcn_fdot2_f32_bf16(wb[i], __builtin_bit_cast(bf16x2_t, xv[i]), v, false);
        }
        v = wave_sum_to_lane63(v);
        total = u == 0 ? v : total + v;
    }
    if (lane == 63 && n_raw < a.N) a.y[n] = (uint16_t)f32_to_bf16_bits(scale * total);
}

//: Wavefronts per workgroup of the whole-row kernel (2, 3, 5, 6 and 8 measured slower:
//: 9728 -> 2560 takes 7.2, 7.5, 7.3, 7.7 and 8.0 us against 6.7).
constexpr int WHOLEROW_WAVES = 4;
//: 16-byte vectors of the activation row per thread: K <= 12288, which three units cannot exceed.
constexpr int WHOLEROW_XV = 6;

template <int CHT, int NU>
int launch_wholerow(const GemvArgs &a, hipStream_t st) {
    const size_t lds = 16 * (size_t)(a.K / 8 + 2);
    const dim3 grid((a.N + WHOLEROW_WAVES - 1) / WHOLEROW_WAVES), block(64 * WHOLEROW_WAVES);
    gemv_w8a16_wholerow_kernel<CHT, NU, WHOLEROW_XV><<<grid, block, lds, st>>>(a);
    return check_launch("cmi_gemv_w8a16");
}

// CMI_E_UNSUPPORTED (no error text) when the shape is not one this kernel takes.
int dispatch_wholerow(const GemvArgs &a, hipStream_t st) {
    if (a.K / 8 > WHOLEROW_XV * 64 * WHOLEROW_WAVES) return CMI_E_UNSUPPORTED;
    if (a.units == 1) {
        // K in one unit: the general kernel is as good or better for small launches (one weight row per
        // wavefront there too, padded activation copy without selects: 4096 -> 2560 3.85 against 3.91 us)
        // and for very tall weights; in between this kernel is 2-4 % faster (2560 -> 19456 9.7 -> 9.4 us,
        // 2560 -> 9728 6.03 -> 5.81 us; two weight rows per wavefront here measured slower again).
        const size_t wbytes = (size_t)a.N * a.K;
        if (wbytes <= ((size_t)20 << 20) || wbytes > ((size_t)128 << 20)) return CMI_E_UNSUPPORTED;
        if (a.unit == 4) return launch_wholerow<4, 1>(a, st);
        if (a.unit == 3) return launch_wholerow<3, 1>(a, st);
        if (a.unit == 2) return launch_wholerow<2, 1>(a, st);
        return CMI_E_UNSUPPORTED;
    }
    if (a.units == 2) {
        if (a.unit == 4) return launch_wholerow<4, 2>(a, st);
        if (a.unit == 3) return launch_wholerow<3, 2>(a, st);
    } else if (a.units == 3) {
        if (a.unit == 4) return launch_wholerow<4, 3>(a, st);
        if (a.unit == 3) return launch_wholerow<3, 3>(a, st);
    }
    return CMI_E_UNSUPPORTED;
}

struct Plan {
    int mt, r, cht, mode;
};

//: Most K-units one launch handles (LDS holds one total per unit and output).
constexpr int MAX_UNITS = 64;
//: Activations up to this many bytes are staged in LDS.
constexpr size_t XLDS_MAX_BYTES = 128 * 1024;

// Blocking is a pure function of (M, N, K); it never changes results.
Plan make_plan(int M, int N, int K) {
    Plan p;
    p.mt = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    const int nseg = (K / 16 + 63) / 64;
    const int unit = unit_segments(nseg);
    const int units = (nseg + unit - 1) / unit;
    // Registers allow 4 chunks per trip for 1-2 rows, 3 for 4 rows (and that only pays
    // when the whole K fits one trip), 1 beyond.
    const int chmax = p.mt <= 2 ? 4 : (p.mt <= 4 && units == 1 && unit <= 3) ? 3 : 1;
    p.cht = unit < chmax ? unit : chmax;
    // balance the sub-trips of a unit (e.g. 4 segments at CHT<=3 -> 2 + 2)
    const int subtrips = (unit + p.cht - 1) / p.cht;
    p.cht = (unit + subtrips - 1) / subtrips;
    p.mode = subtrips > 1 ? 2 : units > 1 ? 1 : 0;
    // Two weight rows per wavefront share the activation fragments.  A single row of a small
    // weight is latency-bound instead: one row per wavefront halves the arithmetic left to do
    // when a wavefront's last bytes arrive (4096 -> 2560: 4.4 -> 4.1 us); from ~20 MB on the
    // launch is throughput-bound and the shared fragments win.
    p.r = (M == 1 && p.mode == 0 && (size_t)N * K <= ((size_t)20 << 20)) ? 1 : 2;
    // Eight rows against a very tall weight (lm_head): four weight rows per wavefront halve the LDS
    // reads of the activation fragments (154 -> 133 us at 2560 -> 151936); on the layer shapes, and
    // at 16 rows (registers), two rows stay faster.
    if (p.mt == 8 && N >= 65536) p.r = 4;
    return p;
}

template <int M, int R, int CHT, int MODE, bool XLDS, int XV>
int launch_xv(const GemvArgs &a, const dim3 grid, const dim3 block, size_t lds, hipStream_t st) {
    static std::atomic<uint64_t> devices{0};
    if (const int rc = reserve_lds(reinterpret_cast<const void *>(gemv_w8a16_kernel<M, R, CHT, MODE, XLDS, XV>),
                                   128 * 1024, devices, "cmi_gemv_w8a16"))
        return rc;
    gemv_w8a16_kernel<M, R, CHT, MODE, XLDS, XV><<<grid, block, lds, st>>>(a);
    return check_launch("cmi_gemv_w8a16");
}

template <int M, int R, int CHT, int MODE, bool XLDS>
int launch(GemvArgs &a, hipStream_t st) {
    a.nblocks = (a.N + R - 1) / R;
    a.subtrips = (a.unit + CHT - 1) / CHT;
    a.xvecs_rcp = (uint32_t)(((1ull << 32) + (a.K / 8) - 1) / (a.K / 8));
    a.uw = a.units < 4 ? a.units : 4;
    a.uw_rcp = (65536u + a.uw - 1) / a.uw;
    a.teams = block_waves(M, MODE, a.units > 1) / a.uw;
    const dim3 grid((a.nblocks + a.teams - 1) / a.teams);
    const dim3 block(64 * a.uw * a.teams);
    const size_t lds = (XLDS ? 16 * (size_t)xlds_vectors(M, a.M, a.K, a.units * a.unit, MODE == 0) : 0) +
                       (MODE == 0 ? 0 : sizeof(float) * a.teams * a.units * R * M);
    if constexpr (XLDS && xstage_short(M) < xstage_vectors(M)) {
        if ((size_t)a.M * (a.K / 8) <= (size_t)xstage_short(M) * block.x)
            return launch_xv<M, R, CHT, MODE, XLDS, xstage_short(M)>(a, grid, block, lds, st);
    }
    return launch_xv<M, R, CHT, MODE, XLDS, xstage_vectors(M)>(a, grid, block, lds, st);
}

// Whether a workgroup of the M-tile's kernel can carry [rows, K] activations into LDS.
bool x_fits_lds(int mt, int rows, int K, int units, int segs, int mode) {
    const size_t xbytes = (size_t)rows * K * 2;                              // carried by the threads
    const size_t ldsbytes = 16 * (size_t)xlds_vectors(mt, rows, K, segs, units == 1);   // held in LDS
    const int uw = units < 4 ? units : 4;
    const int bw = block_waves(mt, mode, units > 1);
    const int xv = mt <= 1 ? xstage_vectors(1) : mt <= 2 ? xstage_vectors(2) : mt <= 4 ? xstage_vectors(4)
                                                                             : xstage_vectors(8);
    const size_t threads = 64 * (size_t)uw * (bw / uw);  // as launch() sizes the workgroup
    // the unit totals share the allocation: one float per (team, unit, weight row, activation row),
    // at most four weight rows per wavefront
    const size_t totals = units > 1 ? sizeof(float) * (bw / uw) * units * 4 * mt : 0;
    return ldsbytes + totals <= XLDS_MAX_BYTES && xbytes <= 16 * (size_t)xv * threads;
}

template <int M, int R, int CHT, int MODE>
int dispatch_lds(GemvArgs &a, hipStream_t st) {
    if (x_fits_lds(M, a.M, a.K, a.units, a.units * a.unit, MODE)) return launch<M, R, CHT, MODE, true>(a, st);
    return launch<M, R, CHT, MODE, false>(a, st);
}

template <int M, int R, int CHT>
int dispatch_x(GemvArgs &a, const Plan &p, hipStream_t st) {
    if (p.mode == 0) return dispatch_lds<M, R, CHT, 0>(a, st);
    if (p.mode == 1) return dispatch_lds<M, R, CHT, 1>(a, st);
    // sub-trips only arise where a unit exceeds the register budget of the M tile
    if constexpr (M >= 4 && CHT == 1) return dispatch_lds<M, R, CHT, 2>(a, st);
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: no sub-trip kernel for M-tile %d, %d chunks", M, CHT);
}

template <int M, int R>
int dispatch_ch(GemvArgs &a, const Plan &p, hipStream_t st) {
    constexpr int CHMAX = M <= 2 ? 4 : M <= 4 ? 3 : 1;
    if (p.cht == 1) return dispatch_x<M, R, 1>(a, p, st);
    if constexpr (CHMAX >= 2) if (p.cht == 2) return dispatch_x<M, R, 2>(a, p, st);
    if constexpr (CHMAX >= 3) if (p.cht == 3) return dispatch_x<M, R, 3>(a, p, st);
    if constexpr (CHMAX >= 4) if (p.cht == 4) return dispatch_x<M, R, 4>(a, p, st);
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: no kernel for M-tile %d with %d chunks", M, p.cht);
}

template <int M>
int dispatch_r(GemvArgs &a, const Plan &p, hipStream_t st) {
    if (p.r == 2) return dispatch_ch<M, 2>(a, p, st);
    if constexpr (M == 1) if (p.r == 1) return dispatch_ch<M, 1>(a, p, st);
    if constexpr (M == 8) if (p.r == 4) return dispatch_ch<M, 4>(a, p, st);
    return fail(CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: no kernel for %d rows per block", p.r);
}

}  // namespace

extern "C" int cmi_gemv_w8a16(const int8_t *wq, const float *ws, const void *x, void *y,
                              int M, int N, int K, void *stream) {
    CMI_REQUIRE(wq && ws && x && y, CMI_E_ARG, "cmi_gemv_w8a16: null pointer");
    CMI_REQUIRE(M >= 1 && M <= 16, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: M=%d outside 1..16", M);
    CMI_REQUIRE(N >= 1 && K >= 16, CMI_E_ARG, "cmi_gemv_w8a16: bad shape N=%d K=%d", N, K);
    CMI_REQUIRE(K % 16 == 0, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: K=%d is not a multiple of 16", K);
    CMI_REQUIRE(aligned(wq, 16) && aligned(x, 16) && aligned(y, 2) && aligned(ws, 4), CMI_E_ARG,
                "cmi_gemv_w8a16: wq and x must be 16-byte aligned");
    const Plan p = make_plan(M, N, K);
    GemvArgs a;
    a.wq = wq;
    a.ws = ws;
    a.x = static_cast<const uint16_t *>(x);
    a.y = static_cast<uint16_t *>(y);
    a.M = M;
    a.N = N;
    a.K = K;
    a.nchunks = K / 16;
    a.nseg = (a.nchunks + 63) / 64;
    a.unit = unit_segments(a.nseg);
    a.units = (a.nseg + a.unit - 1) / a.unit;
    CMI_REQUIRE(a.units <= MAX_UNITS, CMI_E_UNSUPPORTED, "cmi_gemv_w8a16: K=%d above %d", K,
                MAX_UNITS * 4096);
    // Activations too large for LDS: narrower batches fit more often, and rows are
    // independent (same bits whatever the batch), so halve the batch instead.
    if (M > 1 && !x_fits_lds(p.mt, M, K, a.units, a.units * a.unit, p.mode)) {
        const int half = p.mt / 2;
        const int rc = cmi_gemv_w8a16(wq, ws, x, y, half, N, K, stream);
        if (rc != CMI_OK) return rc;
        return cmi_gemv_w8a16(wq, ws, a.x + (size_t)half * K, a.y + (size_t)half * N, M - half, N, K, stream);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    // One row of a long K (two or three units), or of a mid-sized weight with K in one unit: a
    // wavefront per weight row.  CMI_GEMV_WHOLEROW=0 keeps the general kernel (the tests compare
    // the two bit for bit).
    if (M == 1 && p.mode != 2) {
        if (option_gemv_wholerow() != 0) {
            const int rc = dispatch_wholerow(a, st);
            if (rc != CMI_E_UNSUPPORTED) return rc;
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
