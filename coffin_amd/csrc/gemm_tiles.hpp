// Pieces the block-tiled GEMM kernels share: the order in which workgroups take output tiles, the
// widening of a packed int4 weight piece to int8, and the warming of the caches by idle CUs.
#pragma once
#include <cstdint>
#include <hip/hip_runtime.h>

namespace cmi {

// Output tile (tm, tn) of workgroup `id` on a tiles_m x tiles_n grid of tiles.
// Workgroups are dealt round-robin to the 8 XCDs (each with a private L2), so XCD x is given the
// contiguous run of logical tiles [x*per, (x+1)*per); logical tiles walk bands of 8 m tiles,
// m fastest inside a band, so the ~32-64 workgroups an XCD runs at a time form an 8 x (4..8) patch
// that shares its X rows and W rows through that L2 instead of streaming the whole of X once per
// n tile.  A bijection of [0, tiles_m * tiles_n) for every grid.
__device__ __forceinline__ void banded_tile(int tiles_m, int tiles_n, int id, int &tm, int &tn) {
    constexpr int GM = 8;
    const int total = tiles_m * tiles_n;
    int t = id;
    if (total % 8 == 0) t = (id % 8) * (total / 8) + id / 8;
    const int width = GM * tiles_n;
    const int band = t / width, in_band = t - band * width;
    const int first_m = band * GM;
    const int rows = min(tiles_m - first_m, GM);
    tn = in_band / rows;
    tm = first_m + (in_band - tn * rows);
}

// Four codes (0..15, one per byte) -> four int8 (code - 8), no cross-byte borrow.
__device__ __forceinline__ uint32_t rebias4(uint32_t c) {
    return ((c | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

// 16 bytes of the repacked int4 layout (32 codes: within each 32-bit word the low nibbles are
// k 0..3 of that word's 8 and the high nibbles k 4..7) -> 32 int8, `lo` = k 0..15 and
// `hi` = k 16..31 of the piece.
__device__ __forceinline__ void widen_w4_piece(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3,
                                               uint4 &lo, uint4 &hi) {
    lo.x = rebias4(w0 & 0x0F0F0F0Fu);
    lo.y = rebias4((w0 >> 4) & 0x0F0F0F0Fu);
    lo.z = rebias4(w1 & 0x0F0F0F0Fu);
    lo.w = rebias4((w1 >> 4) & 0x0F0F0F0Fu);
    hi.x = rebias4(w2 & 0x0F0F0F0Fu);
    hi.y = rebias4((w2 >> 4) & 0x0F0F0F0Fu);
    hi.z = rebias4(w3 & 0x0F0F0F0Fu);
    hi.w = rebias4((w3 >> 4) & 0x0F0F0F0Fu);
}

// Few tiles: a tile launch is a chain of K / 128 steps, each as long as a CU needs to pull the
// step's operands, and the weight comes from DRAM in 128-byte pieces of 64..128 rows per tile -- a
// third slower than from the memory-side cache (Infinity Cache, 256 MiB, shared by all CUs).  The
// CUs that have no tile therefore read the weight front to back at memory speed and drop it:
// after a few microseconds the tiles' requests are answered by that cache.  (W8A8 tiles: -15..-25 %
// on cold weights.  The W4A8 ring kernels, whose step is set by the widening and the per-group
// flush rather than by the operand stream, measured the same with and without: not used there.)
// Workgroup `part` of `parts` (256 threads each) reads its share of `bytes` (a multiple of 16,
// p 16-byte aligned), eight 16-byte requests in flight per thread.
__device__ __forceinline__ void warm_caches(const void *p, size_t bytes, int part, int parts) {
    const uint4 *v4 = static_cast<const uint4 *>(p);
    const size_t n = bytes / 16;
    const size_t stride = (size_t)parts * 256;
    size_t i = (size_t)part * 256 + threadIdx.x;
    for (; i + 7 * stride < n; i += 8 * stride) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = v4[i + u * stride];
#pragma unroll
        for (int u = 0; u < 8; ++u) asm volatile("" ::"v"(v[u].x), "v"(v[u].y), "v"(v[u].z), "v"(v[u].w));
    }
    for (; i < n; i += stride) {
        const uint4 v = v4[i];
        asm volatile("" ::"v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w));
    }
}

// How many workgroups beyond the `work` that hold tiles read `bytes` of weight through the caches:
// one per CU that would otherwise idle, where at least an eighth of the chip would (32 of them still
// gain 3-7 % at 216..224 tiles, 8..16 nothing), the weight is at most 64 MiB and its 16-byte
// vectors are whole.  (With every CU busy, 32 or 64 such workgroups on top measured faster on some
// shapes and up to 30 % slower on others: not done.)
inline int warm_workgroups(const void *p, size_t bytes, int work) {
    if (work > 224 || bytes > ((size_t)64 << 20) || (reinterpret_cast<uintptr_t>(p) & 15) != 0 || bytes % 16 != 0) return 0;
    return 256 - work;
}

}  // namespace cmi
