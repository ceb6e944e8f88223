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

constexpr int kThreads = 512;  // every GEMM workgroup is 8 wavefronts of 64: two per SIMD
constexpr int kWaves = kThreads / 64;
constexpr int kWave = 64;

// Tile table layout (int32), written by the index build, read by the grouped GEMMs:
//   [0] number of row tiles, [1] rows per tile, [2..3] reserved,
//   then one 4-int entry per row tile: {expert, first tile of that expert,
//   first sorted row of that expert, number of rows of that expert}.
constexpr int kTileHeader = 4;

// Feature-major ("transposed") copies of sorted-row matrices, [feature][padded sorted row]: every
// expert's rows start at a multiple of 32 and are followed by zeros up to the next multiple of
// 32, so that a contraction over an expert's rows can read them in 32-row stages.  Padded
// position of the first sorted row `row0` of expert `e` (momoe_padded_rows() bounds them all):
__host__ __device__ __forceinline__ int padded_start(int row0, int e) { return ((row0 + 31) & ~31) + 32 * e; }

// Index of this wavefront in its workgroup, as a value the compiler knows to be the same in every
// lane: what is derived from it (the rows and columns a wave owns, its share of a transfer) then
// lives in scalar registers instead of taking a vector register per value.
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

struct TileCoord {
  int expert;  // expert index
  int row0;    // first sorted row of this tile
  int prow0;   // padded position of that row
  int rows;    // valid rows in this tile (1..rows per tile)
  int tn;      // column block
  int mbase;   // first tile row owned by this wave (waves 0-3 / 4-7 split the tile's rows)
  int na;      // 32-row fragment rows owned by this wave (0..5)
  bool valid;
};

// Persistent-workgroup iterator over the (row tile, column block) pairs of a grouped GEMM.
// Workgroups are dealt round-robin to the 8 XCDs, so id%8 selects the XCD; each XCD owns one
// contiguous eighth of the tile sequence (expert-major; the order inside an expert is given at resolve()) and its
// workgroups walk it with a stride of gridDim/8.  All tiles of an expert therefore run on
// one XCD close together in time and share its L2 for both the expert's weights and its
// token rows.
// A tile is looked up in two steps so that the table read can travel while other work runs:
// fetch() issues the scalar loads of the workgroup's next tile, resolve() does the arithmetic.
struct TileSched {
  static constexpr int kBandTiles = 4;
  // tile height the table was built for
  static __device__ __forceinline__ int tile_rows_of(const int* table) {
    return *(const int __attribute__((address_space(4)))*)(table + 1);
  }
  struct Raw {
    int q, expert, first, rstart, mi;
    bool any;
  };
  const int* table;
  int nb, bm, begin, total, chunk, xcd, pos, stride;

  // tiles before row tile `first_row_tile` (all its column blocks) are left out; a table whose
  // tiles are taller than the kernel's `max_tile_rows` yields no tiles at all
  __device__ __forceinline__ TileSched(const int* table_, int nb_, int max_tile_rows,
                                       int first_row_tile = 0)
      : table(table_), nb(nb_) {
    bm = *(const int __attribute__((address_space(4)))*)(table + 1);
    const int ntiles = bm <= max_tile_rows ? *(const int __attribute__((address_space(4)))*)table : 0;
    begin = min(first_row_tile, ntiles) * nb;
    total = ntiles * nb;
    chunk = (total - begin + 7) >> 3;
    xcd = blockIdx.x & 7;
    pos = blockIdx.x >> 3;
    stride = gridDim.x >> 3;
  }
  __device__ __forceinline__ Raw fetch() {
    Raw r;
    r.any = false;
    if (pos >= chunk) return r;
    const int q = begin + xcd * chunk + pos;
    pos += stride;
    if (q >= total) return r;
    const int __attribute__((address_space(4)))* e =
        (const int __attribute__((address_space(4)))*)(table + kTileHeader + 4 * (q / nb));
    r.q = q;
    r.expert = e[0];
    r.first = e[1];
    r.rstart = e[2];
    r.mi = e[3];
    r.any = true;
    return r;
  }
  __device__ __forceinline__ TileCoord resolve(const Raw& r) const {
    TileCoord tc;
    tc.valid = r.any;
    if (!r.any) return tc;
    // The expert's rows are 32-row fragment rows, dealt to its nt row tiles as evenly as they
    // go (the first few tiles hold one more), not full tiles plus a remainder: tiles that share
    // a weight block then take nearly equally long and stay in step, no tile streams a whole
    // weight block for a handful of rows, and only the expert's last fragment row is ragged.
    const int nt = (r.mi + bm - 1) / bm;
    const int nfe = (r.mi + 31) >> 5, fbase = nfe / nt, fextra = nfe - fbase * nt;
    // Order inside an expert: bands of kBandTiles row tiles, each band crossing every column
    // block before the next band starts (row tile fastest inside a band).  The workgroups of
    // an XCD hold consecutive positions at any moment, so they share a few row tiles and a few
    // weight blocks in L2 however many rows the expert has.
    const int qq = r.q - r.first * nb;
    const int band = qq / (kBandTiles * nb);
    const int in_band = qq - band * (kBandTiles * nb);
    const int band_rows = min(kBandTiles, nt - band * kBandTiles);
    const int tl = band * kBandTiles + in_band % band_rows;
    tc.tn = in_band / band_rows;
    tc.expert = r.expert;
    const int f0 = tl * fbase + min(tl, fextra);  // first fragment row of this tile
    tc.row0 = r.rstart + 32 * f0;
    tc.prow0 = padded_start(r.rstart, r.expert) + 32 * f0;
    tc.rows = min(32 * (fbase + (tl < fextra ? 1 : 0)), r.mi - 32 * f0);
    // the tile's fragment rows are dealt to the two wave rows as evenly as possible
    const int nf = (tc.rows + 31) >> 5, half = (nf + 1) >> 1;
    const bool upper = wave_id() >= kWaves / 2;
    tc.mbase = upper ? 32 * half : 0;
    tc.na = upper ? nf - half : half;
    return tc;
  }
  __device__ __forceinline__ TileCoord next() { return resolve(fetch()); }
  // first row tile of the expert that holds sorted row `row` (number of row tiles if the row
  // lies past the last expert): everything before it only has rows below `row`
  static __device__ __forceinline__ int expert_tile_of_row(const int* table, int64_t row) {
    const int ntiles = *(const int __attribute__((address_space(4)))*)table;
    int lo = 0, hi = ntiles;  // experts of the row tiles before lo end at or below `row`
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      const int __attribute__((address_space(4)))* e =
          (const int __attribute__((address_space(4)))*)(table + kTileHeader + 4 * mid);
      if ((int64_t)e[2] + e[3] <= row) lo = mid + 1; else hi = mid;
    }
    if (lo >= ntiles) return ntiles;
    return *(const int __attribute__((address_space(4)))*)(table + kTileHeader + 4 * lo + 1);
  }
};

__device__ __forceinline__ float bf2f(bf16 v) { return (float)v; }
__device__ __forceinline__ bf16 f2bf(float v) { return (bf16)v; }

// 1 / (1 + e^-v) with the hardware reciprocal (1 ulp): a plain `1.0f / x` compiles to the
// correctly rounded division, ten instructions where the results are rounded to bf16 anyway
__device__ __forceinline__ float sigmoidf_fast(float v) {
  return __builtin_amdgcn_rcpf(1.0f + __expf(-v));
}

// Measurement aid (momoe_set_clock_trace): while a trace buffer is set, one wavefront of every
// grouped-GEMM launch adds the shader-clock ticks it ran for to buf[0] and the ticks of the
// constant 100 MHz counter over the same interval to buf[1]; 100 * buf[0] / buf[1] is the
// average shader clock in MHz while those kernels ran.
unsigned long long* clock_trace_buffer();  // host side: the buffer in use, or nullptr
struct ClockTrace {
  unsigned long long* buf;
  // start: subtract the counters, finish(): add them -- nothing is kept in registers in between
  __device__ __forceinline__ explicit ClockTrace(unsigned long long* b) : buf(b) {
    if (active()) {
      atomicAdd(buf, 0ull - (unsigned long long)clock64());
      atomicAdd(buf + 1, 0ull - (unsigned long long)wall_clock64());
    }
  }
  __device__ __forceinline__ bool active() const {
    return buf != nullptr && blockIdx.x == 0 && threadIdx.x == 0;
  }
  __device__ __forceinline__ void finish() const {
    if (active()) {
      atomicAdd(buf, (unsigned long long)clock64());
      atomicAdd(buf + 1, (unsigned long long)wall_clock64());
    }
  }
};

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? MOMOE_OK : MOMOE_ERR_LAUNCH;
}

inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// upper bound on the number of row tiles for any routing with msum pairs over n experts
inline int64_t max_row_tiles(int64_t msum, int64_t n, int64_t bm) { return msum / bm + n; }

}  // namespace momoe
