// 16-row x 128-byte operand tiles for the v_mfma_i32_16x16x64_i8 small-batch
// kernels.  The MFMA wants lane l to hold 16 bytes of row l%16, which as a load
// pattern touches half a cache line of each of 16 rows per instruction and
// measured 30 % slower than whole lines.  So a tile is fetched as two loads of
// 8 rows x 128 bytes (lane l: row l/8, 16-byte piece l%8) and turned into the
// MFMA arrangement through a wavefront-private LDS patch: LDS executes one
// wavefront's instructions in order, so no barrier is involved.
#pragma once
#include "common.hpp"

namespace cmi {
namespace rows16 {

typedef int v4i32 __attribute__((ext_vector_type(4)));

constexpr int TILE_PITCH = 144;             // 128 + 16: the 16 rows of a column read hit 16 different bank groups
constexpr int PATCH_BYTES = 16 * TILE_PITCH;

// Global side: byte offset of this lane's piece in the half tile `half` (rows 8*half ..) of the
// line starting at byte `line_byte` of each row; rows clamped to `last_row`.  CLAMP: also keep
// the piece inside a row of `row_bytes` (rows that end in the middle of a line).
template <bool CLAMP = false>
__device__ __forceinline__ size_t tile_src(int lane, int half, int first_row, int last_row, size_t row_bytes,
                                           int line_byte) {
    const int row = min(first_row + 8 * half + (lane >> 3), last_row);
    int off = line_byte + (lane & 7) * 16;
    if (CLAMP) off = min(off, (int)row_bytes - 16);
    return (size_t)row * row_bytes + off;
}

// Park both halves of a tile in the patch.
__device__ __forceinline__ void tile_park(uint8_t *patch, int lane, v4i32 lo, v4i32 hi) {
    uint8_t *p = patch + (lane >> 3) * TILE_PITCH + (lane & 7) * 16;
    *reinterpret_cast<v4i32 *>(p) = lo;
    *reinterpret_cast<v4i32 *>(p + 8 * TILE_PITCH) = hi;
}

// Piece `piece` (0..7) of row lane%16.
__device__ __forceinline__ v4i32 tile_take(const uint8_t *patch, int lane, int piece) {
    return *reinterpret_cast<const v4i32 *>(patch + (lane & 15) * TILE_PITCH + piece * 16);
}

}  // namespace rows16
}  // namespace cmi
