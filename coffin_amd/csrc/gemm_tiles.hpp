// Pieces the block-tiled GEMM kernels share: the order in which workgroups take output tiles, and
// the widening of a packed int4 weight piece to int8.
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

}  // namespace cmi
