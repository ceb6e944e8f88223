// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/momoe_hip.h"

namespace momoe {

typedef __bf16 bf16;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;  // every GEMM workgroup is 4 wavefronts of 64
constexpr int kWave = 64;

// Tile table layout (int32), written by the index build, read by the grouped GEMMs:
//   [0] number of row tiles, [1] rows per tile, [2..3] reserved,
//   then one 4-int entry per row tile: {expert, first tile of that expert,
//   first sorted row of that expert, number of rows of that expert}.
constexpr int kTileHeader = 4;

struct TileCoord {
  int expert;  // expert index
  int row0;    // first sorted row of this tile
  int rows;    // valid rows in this tile (1..rows per tile)
  int tn;      // column block
  bool valid;
};

// Map the linear workgroup id to a (row tile, column block).  Workgroups are dealt
// round-robin to the 8 XCDs, so id%8 selects the XCD; each XCD walks one contiguous
// eighth of the (expert-major, column-block, row-tile-minor) sequence.  All tiles of
// an expert therefore run on one XCD close together in time and share its L2 for
// both the expert's weights and its token rows.
__device__ __forceinline__ TileCoord decode_tile(const int* __restrict__ table, int nb) {
  TileCoord tc;
  tc.valid = false;
  const int ntiles = table[0];
  const int bm = table[1];
  const int total = ntiles * nb;
  const int chunk = (total + 7) >> 3;
  const int bid = blockIdx.x;
  const int xcd = bid & 7, slot = bid >> 3;
  if (slot >= chunk) return tc;
  const int q = xcd * chunk + slot;
  if (q >= total) return tc;
  const int* e = table + kTileHeader + 4 * (q / nb);
  const int expert = e[0], first = e[1], rstart = e[2], mi = e[3];
  const int nt = (mi + bm - 1) / bm;
  const int qq = q - first * nb;
  const int tl = qq % nt;
  tc.tn = qq / nt;
  tc.expert = expert;
  tc.row0 = rstart + tl * bm;
  tc.rows = min(bm, mi - tl * bm);
  tc.valid = true;
  return tc;
}

__device__ __forceinline__ float bf2f(bf16 v) { return (float)v; }
__device__ __forceinline__ bf16 f2bf(float v) { return (bf16)v; }

__device__ __forceinline__ float sigmoidf_fast(float v) { return 1.0f / (1.0f + __expf(-v)); }

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? MOMOE_OK : MOMOE_ERR_LAUNCH;
}

inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// upper bound on the number of row tiles for any routing with msum pairs over n experts
inline int64_t max_row_tiles(int64_t msum, int64_t n, int64_t bm) { return msum / bm + n; }

}  // namespace momoe
