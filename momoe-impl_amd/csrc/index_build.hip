// Routing index build: expert histogram, prefix sums, sorted-row scatter and
// the device-side tile table.  Integer work, HBM/latency bound: the mask is read
// twice with coalesced loads, positions come from wavefront ballots.
//
// Decomposition: the [N, M] mask is cut into panels of 16 experts x 256 tokens;
// one workgroup (256 lanes = 256 tokens) owns a panel.
//   pass 1 (count):   per panel, tokens per expert (ballot + popcount) and set
//                     bits per token.
//   pass 2 (scan):    one workgroup: per-expert exclusive scan over panels,
//                     exclusive scan over experts (cumsums), tile table.
//   pass 3 (scatter): per panel, each set bit learns its sorted row
//                     (expert base + panel base + wave base + rank in ballot) and
//                     its slot (set bits of the token in earlier experts).
#include <mutex>

#include "common.hpp"

namespace momoe {
namespace {

constexpr int kPanelTokens = 256;
constexpr int kPanelExperts = 16;
constexpr int kMaxExperts = 4096;

// The 16 mask entries of token m in expert group g, as a bit set.  Loads are unconditional (row
// and column clamped into the matrix, the result masked afterwards): a load under a branch is
// waited for before the next one is issued, which made this function one memory latency PER
// ENTRY instead of one per group.
__device__ __forceinline__ uint32_t load_panel_bits(const int32_t* __restrict__ mask, int64_t sn,
                                                    int64_t sm, int M, int N, int g, int m) {
  const int32_t* col = mask + (int64_t)min(m, M - 1) * sm;
  int32_t v[kPanelExperts];
#pragma unroll
  for (int e = 0; e < kPanelExperts; ++e)
    v[e] = col[(int64_t)min(g * kPanelExperts + e, N - 1) * sn];
  uint32_t bits = 0;
#pragma unroll
  for (int e = 0; e < kPanelExperts; ++e)
    bits |= (v[e] != 0 && g * kPanelExperts + e < N ? 1u : 0u) << e;
  return m < M ? bits : 0u;
}

__global__ __launch_bounds__(kPanelTokens) void index_count_kernel(
    const int32_t* __restrict__ mask, int64_t sn, int64_t sm, int M, int N, int NC,
    int32_t* __restrict__ part /*[N][NC]*/, int32_t* __restrict__ tokcnt /*[NG][M]*/) {
  __shared__ int32_t wcnt[kPanelExperts][4];
  const int c = blockIdx.x, g = blockIdx.y;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int m = c * kPanelTokens + t;
  const uint32_t bits = load_panel_bits(mask, sn, sm, M, N, g, m);
#pragma unroll
  for (int e = 0; e < kPanelExperts; ++e) {
    const uint64_t b = __ballot((bits >> e) & 1u);
    if (lane == 0) wcnt[e][wave] = __popcll(b);
  }
  if (m < M) tokcnt[(int64_t)g * M + m] = __popc(bits);
  __syncthreads();
  if (t < kPanelExperts) {
    const int i = g * kPanelExperts + t;
    if (i < N) part[(int64_t)i * NC + c] = wcnt[t][0] + wcnt[t][1] + wcnt[t][2] + wcnt[t][3];
  }
}

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int o = __shfl_up(v, d);
    if (lane >= d) v += o;
  }
  return v;
}

// Tile height for a routing (tile_rows = 0 asked for it).  A row tile streams its rows and a
// 256-column block of the expert's weights, so a GEMM's time goes with the sum over the tiles of
// (rows + 256): an expert of v rows costs v + 256 * (number of its tiles).  Tall tiles save whole
// passes over the weights (an expert of 513..640 rows: two instead of three) but their kernels
// are a few percent less efficient per tile: they are taken when they save more than 4 %.
__device__ __forceinline__ int choose_tile_rows(const int32_t* sizes, int N, int lane) {
  int64_t c_std = 0, c_tall = 0;
  for (int i = lane; i < N; i += 64) {
    const int v = sizes[i];
    c_std += v + 256 * ((v + MOMOE_RECOMPUTE_TILE_ROWS - 1) / MOMOE_RECOMPUTE_TILE_ROWS);
    c_tall += v + 256 * ((v + MOMOE_TILE_ROWS - 1) / MOMOE_TILE_ROWS);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    c_std += __shfl_xor(c_std, o);
    c_tall += __shfl_xor(c_tall, o);
  }
  return c_tall * 26 < c_std * 25 ? MOMOE_TILE_ROWS : MOMOE_RECOMPUTE_TILE_ROWS;
}

__global__ __launch_bounds__(1024) void index_scan_kernel(
    int32_t* __restrict__ part, int N, int NC, int64_t msum_cap,
    int64_t* __restrict__ sizes, int32_t* __restrict__ cumsums,
    int32_t* __restrict__ table, int tile_rows_arg, int32_t* __restrict__ table_rc,
    int32_t* __restrict__ violations, int32_t* __restrict__ idx, int32_t* __restrict__ which) {
  __shared__ int32_t s_size[kMaxExperts];
  __shared__ int32_t s_cum[kMaxExperts];
  __shared__ int32_t s_first[kMaxExperts];
  __shared__ int32_t s_total[3];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  // per expert: exclusive scan of the panel counts, in place
  for (int i = wave; i < N; i += 16) {
    int running = 0;
    for (int c0 = 0; c0 < NC; c0 += 64) {
      const int c = c0 + lane;
      const int v = c < NC ? part[(int64_t)i * NC + c] : 0;
      const int inc = wave_inclusive_scan(v, lane);
      if (c < NC) part[(int64_t)i * NC + c] = running + inc - v;
      running += __shfl(inc, 63);
    }
    if (lane == 0) s_size[i] = running;
  }
  __syncthreads();
  if (wave == 0) {
    const int tile_rows = tile_rows_arg > 0 ? tile_rows_arg : choose_tile_rows(s_size, N, lane);
    int run_rows = 0, run_tiles = 0;
    for (int i0 = 0; i0 < N; i0 += 64) {
      const int i = i0 + lane;
      const int v = i < N ? s_size[i] : 0;
      const int nt = (v + tile_rows - 1) / tile_rows;
      const int inc = wave_inclusive_scan(v, lane);
      const int inct = wave_inclusive_scan(nt, lane);
      if (i < N) {
        s_cum[i] = run_rows + inc - v;
        s_first[i] = run_tiles + inct - nt;
        cumsums[i] = run_rows + inc - v;
        sizes[i] = (int64_t)v;
      }
      run_rows += __shfl(inc, 63);
      run_tiles += __shfl(inct, 63);
    }
    if (lane == 0) {
      cumsums[N] = run_rows;
      const bool overflow = (int64_t)run_rows > msum_cap;
      if (overflow) atomicAdd(violations, 1);
      s_total[0] = overflow ? 0 : run_tiles;
      s_total[1] = run_rows;
      s_total[2] = tile_rows;
      table[0] = overflow ? 0 : run_tiles;
      table[1] = tile_rows;
      table[2] = 0;
      table[3] = 0;
    }
  }
  __syncthreads();
  // A routing with fewer than M*K pairs leaves the sorted rows past the last pair without a
  // token: give them token 0 / slot 0, so that nothing downstream reads an undefined id.
  for (int64_t r = (int64_t)s_total[1] + t; r < msum_cap; r += 1024) {
    idx[r] = 0;
    which[r] = 0;
  }
  const int tile_rows = s_total[2];
  // the second table (tiles of the recomputing GEMM's height) is the same table when that is the
  // height chosen; otherwise the row tiles are counted again below
  const bool same = tile_rows == MOMOE_RECOMPUTE_TILE_ROWS;
  if (s_total[0] == 0) {
    if (table_rc != nullptr && t < kTileHeader) table_rc[t] = t == 1 ? MOMOE_RECOMPUTE_TILE_ROWS : 0;
    return;
  }
  auto write_entries = [&](int32_t* dst, int rows) {
    for (int i = t; i < N; i += 1024) {
      const int v = s_size[i];
      const int nt = (v + rows - 1) / rows;
      const int first = s_first[i];
      for (int k = 0; k < nt; ++k) {
        int32_t* e = dst + kTileHeader + 4 * (first + k);
        e[0] = i;
        e[1] = first;
        e[2] = s_cum[i];
        e[3] = v;
      }
    }
  };
  write_entries(table, tile_rows);
  if (table_rc == nullptr) return;
  if (same) {
    write_entries(table_rc, tile_rows);
    if (t < kTileHeader) table_rc[t] = t == 0 ? s_total[0] : t == 1 ? tile_rows : 0;
    return;
  }
  __syncthreads();  // every thread has read s_first
  if (wave == 0) {
    int run_tiles = 0;
    for (int i0 = 0; i0 < N; i0 += 64) {
      const int i = i0 + lane;
      const int v = i < N ? s_size[i] : 0;
      const int nt = (v + MOMOE_RECOMPUTE_TILE_ROWS - 1) / MOMOE_RECOMPUTE_TILE_ROWS;
      const int inct = wave_inclusive_scan(nt, lane);
      if (i < N) s_first[i] = run_tiles + inct - nt;
      run_tiles += __shfl(inct, 63);
    }
    if (lane < kTileHeader) table_rc[lane] = lane == 0 ? run_tiles : lane == 1 ? MOMOE_RECOMPUTE_TILE_ROWS : 0;
  }
  __syncthreads();
  write_entries(table_rc, MOMOE_RECOMPUTE_TILE_ROWS);
}

__global__ __launch_bounds__(kPanelTokens) void index_scatter_kernel(
    const int32_t* __restrict__ mask, int64_t sn, int64_t sm, int M, int N, int K, int NC,
    const int32_t* __restrict__ part, const int32_t* __restrict__ tokcnt,
    const int32_t* __restrict__ cumsums, int32_t* __restrict__ idx, int32_t* __restrict__ which,
    int32_t* __restrict__ inv, int32_t* __restrict__ violations) {
  __shared__ int32_t wcnt[kPanelExperts][4];
  const int c = blockIdx.x, g = blockIdx.y;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int m = c * kPanelTokens + t;
  const int64_t msum = (int64_t)M * K;
  const bool overflow = (int64_t)cumsums[N] > msum;
  const uint32_t bits = load_panel_bits(mask, sn, sm, M, N, g, m);
  uint64_t ballots[kPanelExperts];
#pragma unroll
  for (int e = 0; e < kPanelExperts; ++e) {
    ballots[e] = __ballot((bits >> e) & 1u);
    if (lane == 0) wcnt[e][wave] = __popcll(ballots[e]);
  }
  int k = 0;
  if (m < M)
    for (int gg = 0; gg < g; ++gg) k += tokcnt[(int64_t)gg * M + m];
  __syncthreads();
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int e = 0; e < kPanelExperts; ++e) {
    const int i = g * kPanelExperts + e;
    if (i >= N) break;
    if ((bits >> e) & 1u) {
      int woff = 0;
      for (int w = 0; w < wave; ++w) woff += wcnt[e][w];
      const int64_t row = (int64_t)cumsums[i] + part[(int64_t)i * NC + c] + woff +
                          __popcll(ballots[e] & below);
      if (row < msum) {
        idx[row] = m;
        which[row] = k;
      }
      // more pairs than rows: the GEMMs get an empty tile table and write nothing, so no token
      // may point at a row (the combine then gives zeros instead of unwritten memory)
      if (k < K) inv[(int64_t)m * K + k] = row < msum && !overflow ? (int32_t)row : -1;
      ++k;
    }
  }
  if (m < M && g == gridDim.y - 1 && k != K) {
    atomicAdd(violations, 1);
    // slots the token does not fill: -1 = "no row" (momoe_combine skips them)
    for (int kk = k; kk < K; ++kk) inv[(int64_t)m * K + kk] = -1;
  }
}

// The whole index build in one launch of one workgroup, for at most 256 tokens (one token
// panel) and 256 experts: decode-sized calls, where three dependent launches cost more than
// the work.  Thread t is token t and reads its whole mask column up front (all loads in flight
// at once: one memory latency), as 16 bits per group of 16 experts; one ballot per expert gives
// the lane masks of its tokens, a scan over the experts gives cumsums and the tile table, and
// every token then places its own K pairs from its bits and those masks.
// the single-launch kernels: one expert's entries, and the header, in the table and (if asked
// for) in its copy for the recomputing GEMM
__device__ __forceinline__ void write_tile_entries(int32_t* table, int32_t* table_rc, int first,
                                                   int nt, int expert, int row0, int rows) {
  for (int k = 0; k < nt; ++k) {
    int32_t* e = table + kTileHeader + 4 * (first + k);
    e[0] = expert;
    e[1] = first;
    e[2] = row0;
    e[3] = rows;
    if (table_rc != nullptr) {
      int32_t* c = table_rc + kTileHeader + 4 * (first + k);
      c[0] = expert;
      c[1] = first;
      c[2] = row0;
      c[3] = rows;
    }
  }
}
__device__ __forceinline__ void write_tile_header(int32_t* table, int32_t* table_rc, int ntiles,
                                                  int tile_rows) {
  table[0] = ntiles;
  table[1] = tile_rows;
  table[2] = 0;
  table[3] = 0;
  if (table_rc != nullptr) {
    table_rc[0] = ntiles;
    table_rc[1] = tile_rows;
    table_rc[2] = 0;
    table_rc[3] = 0;
  }
}

constexpr int kSmallMaxGroups = 16;
constexpr int kSmallMaxExperts = kSmallMaxGroups * kPanelExperts;

template <int NGROUPS>
__global__ __launch_bounds__(kPanelTokens) void index_small_kernel(
    const int32_t* __restrict__ mask, int64_t sn, int64_t sm, int M, int N, int K,
    int64_t* __restrict__ sizes, int32_t* __restrict__ cumsums, int32_t* __restrict__ idx,
    int32_t* __restrict__ which, int32_t* __restrict__ inv, int32_t* __restrict__ table,
    int tile_rows_arg, int32_t* __restrict__ table_rc, int32_t* __restrict__ violations) {
  // asked to choose the tile height: with at most 256 tokens no expert holds more than 256 rows,
  // and taller tiles save nothing.  table_rc (only with that choice) receives the same table.
  const int tile_rows = tile_rows_arg > 0 ? tile_rows_arg : MOMOE_RECOMPUTE_TILE_ROWS;
  static_assert(kPanelTokens <= MOMOE_RECOMPUTE_TILE_ROWS, "one tile per expert in the one-launch kernel");
  __shared__ uint64_t ball[NGROUPS * kPanelExperts][4];  // tokens of expert i in wave w, as a lane mask
  __shared__ int32_t s_base[NGROUPS * kPanelExperts][4];  // sorted row of expert i's first token in wave w
  __shared__ int32_t s_wave[4][2];
  static_assert(NGROUPS % 4 == 0, "the experts of a token are walked as 64-bit words");
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int64_t msum = (int64_t)M * K;
  uint32_t bits[NGROUPS];
#pragma unroll
  for (int g = 0; g < NGROUPS; ++g) bits[g] = load_panel_bits(mask, sn, sm, M, N, g, t);
#pragma unroll
  for (int g = 0; g < NGROUPS; ++g)
#pragma unroll
    for (int e = 0; e < kPanelExperts; ++e) {
      const uint64_t b = __ballot((bits[g] >> e) & 1u);
      if (lane == 0) ball[g * kPanelExperts + e][wave] = b;
    }
  __syncthreads();
  // exclusive scan over the experts of (rows, row tiles): one expert per thread
  const int v = t < N ? __popcll(ball[t][0]) + __popcll(ball[t][1]) + __popcll(ball[t][2]) + __popcll(ball[t][3]) : 0;
  const int nt = (v + tile_rows - 1) / tile_rows;
  const int irows = wave_inclusive_scan(v, lane), itiles = wave_inclusive_scan(nt, lane);
  if (lane == 63) {
    s_wave[wave][0] = irows;
    s_wave[wave][1] = itiles;
  }
  __syncthreads();
  int brow = irows - v, btile = itiles - nt;
  for (int w = 0; w < wave; ++w) {
    brow += s_wave[w][0];
    btile += s_wave[w][1];
  }
  const int total = s_wave[0][0] + s_wave[1][0] + s_wave[2][0] + s_wave[3][0];
  const int total_tiles = s_wave[0][1] + s_wave[1][1] + s_wave[2][1] + s_wave[3][1];
  const bool overflow = (int64_t)total > msum;
  if (t < N) {
    int run = brow;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      s_base[t][w] = run;
      run += __popcll(ball[t][w]);
    }
    cumsums[t] = brow;
    sizes[t] = (int64_t)v;
    if (!overflow) write_tile_entries(table, table_rc, btile, nt, t, brow, v);
  }
  if (t == 0) {
    cumsums[N] = total;
    if (overflow) atomicAdd(violations, 1);
    write_tile_header(table, table_rc, overflow ? 0 : total_tiles, tile_rows);
  }
  // sorted rows past the last pair (a routing with fewer than M*K pairs): token 0, slot 0
  for (int64_t r = (int64_t)total + t; r < msum; r += kPanelTokens) {
    idx[r] = 0;
    which[r] = 0;
  }
  __syncthreads();
  // every token walks its own pairs (K of them, not N candidates), lowest expert first: one loop
  // over all of its experts, so that a wavefront makes as many rounds as its busiest token has
  // pairs (a loop per group of 16 experts made the sum over the groups of that maximum)
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  constexpr int NWORDS = NGROUPS / 4;
  uint64_t word[NWORDS];
#pragma unroll
  for (int j = 0; j < NWORDS; ++j)
    word[j] = (uint64_t)bits[4 * j] | ((uint64_t)bits[4 * j + 1] << 16) |
              ((uint64_t)bits[4 * j + 2] << 32) | ((uint64_t)bits[4 * j + 3] << 48);
  int k = 0;
  for (;;) {
    int i = -1;
#pragma unroll
    for (int j = NWORDS - 1; j >= 0; --j)
      if (word[j] != 0) i = 64 * j + __ffsll((unsigned long long)word[j]) - 1;
    if (i < 0) break;
#pragma unroll
    for (int j = 0; j < NWORDS; ++j)
      if ((i >> 6) == j) word[j] &= word[j] - 1;
    const int64_t row = (int64_t)s_base[i][wave] + __popcll(ball[i][wave] & below);
    if (row < msum) {
      idx[row] = t;
      which[row] = k;
    }
    if (k < K) inv[(int64_t)t * K + k] = row < msum && !overflow ? (int32_t)row : -1;
    ++k;
  }
  if (t < M && k != K) {
    atomicAdd(violations, 1);
    for (int kk = k; kk < K; ++kk) inv[(int64_t)t * K + kk] = -1;
  }
}

// The same for at most 64 tokens, the other way round: thread e is EXPERT e and holds its row of
// the mask as a 64-bit set of tokens.  Transposing the mask costs one ballot per token here (at
// most 64) instead of one per expert (128 to 256 in the kernel above), a thread loads M mask
// entries instead of N, and an expert has its few rows placed in as many rounds: a 16-token call
// has its index in a third of the time (5.7 us against 16.5 at 128 experts).
// MCH = ceil(M / 16): all of a thread's mask loads are in flight at once.
constexpr int kTinyTokens = 64;
template <int MCH>
__global__ __launch_bounds__(kPanelTokens) void index_tiny_kernel(
    const int32_t* __restrict__ mask, int64_t sn, int64_t sm, int M, int N, int K,
    int64_t* __restrict__ sizes, int32_t* __restrict__ cumsums, int32_t* __restrict__ idx,
    int32_t* __restrict__ which, int32_t* __restrict__ inv, int32_t* __restrict__ table,
    int tile_rows_arg, int32_t* __restrict__ table_rc, int32_t* __restrict__ violations,
    bool rows_of_int4) {
  static_assert(MCH >= 1 && 16 * MCH <= kTinyTokens, "token chunks of 16");
  const int tile_rows = tile_rows_arg > 0 ? tile_rows_arg : MOMOE_RECOMPUTE_TILE_ROWS;
  __shared__ uint64_t tokb[kTinyTokens][4];  // experts of token m among the experts of wave w, as a lane mask
  __shared__ int32_t s_slot[kTinyTokens][4];  // pairs of token m held by the experts of the waves below w
  __shared__ int32_t s_wave[4][2];
  const int e = threadIdx.x, lane = e & 63, wave = e >> 6;
  const int64_t msum = (int64_t)M * K;
  // the expert's row of the mask as a bit set; loads unconditional, row and column clamped
  uint64_t bits = 0;
  const int32_t* row = mask + (int64_t)min(e, N - 1) * sn;
  if (rows_of_int4) {
    // contiguous rows of a multiple of 4 tokens, 16-byte aligned (checked on the host): four
    // tokens per load.  Lanes read rows that lie apart, so a load instruction costs one line
    // request per lane whatever its width, and this path makes a quarter of them.
    int4 v[4 * MCH];
#pragma unroll
    for (int c = 0; c < 4 * MCH; ++c) v[c] = ((const int4*)row)[min(c, M / 4 - 1)];
#pragma unroll
    for (int c = 0; c < 4 * MCH; ++c) {
      const uint64_t nib = (v[c].x != 0 ? 1u : 0u) | (v[c].y != 0 ? 2u : 0u) | (v[c].z != 0 ? 4u : 0u) |
                           (v[c].w != 0 ? 8u : 0u);
      if (4 * c < M) bits |= nib << (4 * c);
    }
  } else {
    int32_t v[16 * MCH];
#pragma unroll
    for (int m = 0; m < 16 * MCH; ++m) v[m] = row[(int64_t)min(m, M - 1) * sm];
#pragma unroll
    for (int m = 0; m < 16 * MCH; ++m) bits |= (uint64_t)(v[m] != 0 && m < M ? 1 : 0) << m;
  }
  if (e >= N) bits = 0;
  // per token: the experts that hold it
  for (int m = 0; m < M; ++m) {
    const uint64_t b = __ballot((bits >> m) & 1ull);
    if (lane == 0) tokb[m][wave] = b;
  }
  // exclusive scan over the experts of (rows, row tiles)
  const int v = __popcll(bits);
  const int nt = (v + tile_rows - 1) / tile_rows;
  const int irows = wave_inclusive_scan(v, lane), itiles = wave_inclusive_scan(nt, lane);
  if (lane == 63) {
    s_wave[wave][0] = irows;
    s_wave[wave][1] = itiles;
  }
  __syncthreads();
  int brow = irows - v, btile = itiles - nt;
  for (int w = 0; w < wave; ++w) {
    brow += s_wave[w][0];
    btile += s_wave[w][1];
  }
  const int total = s_wave[0][0] + s_wave[1][0] + s_wave[2][0] + s_wave[3][0];
  const int total_tiles = s_wave[0][1] + s_wave[1][1] + s_wave[2][1] + s_wave[3][1];
  const bool overflow = (int64_t)total > msum;
  if (e < N) {
    cumsums[e] = brow;
    sizes[e] = (int64_t)v;
    if (!overflow) write_tile_entries(table, table_rc, btile, nt, e, brow, v);
  }
  if (e == 0) {
    cumsums[N] = total;
    if (overflow) atomicAdd(violations, 1);
    write_tile_header(table, table_rc, overflow ? 0 : total_tiles, tile_rows);
  }
  // sorted rows past the last pair (a routing with fewer than M*K pairs): token 0, slot 0
  for (int64_t r = (int64_t)total + e; r < msum; r += kPanelTokens) {
    idx[r] = 0;
    which[r] = 0;
  }
  // thread m counts the pairs of token m
  int pairs = 0;
  if (e < M) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      s_slot[e][w] = pairs;
      pairs += __popcll(tokb[e][w]);
    }
  }
  __syncthreads();
  // the expert places its pairs, lowest token first; the slot of a pair within its token is the
  // number of lower-numbered experts that hold the token
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  uint64_t rest = bits;
  for (int r = 0; rest != 0; ++r) {
    const int m = __ffsll((unsigned long long)rest) - 1;
    rest &= rest - 1;
    const int k = s_slot[m][wave] + __popcll(tokb[m][wave] & below);
    const int64_t srow = (int64_t)brow + r;
    if (srow < msum) {
      idx[srow] = m;
      which[srow] = k;
    }
    if (k < K) inv[(int64_t)m * K + k] = srow < msum && !overflow ? (int32_t)srow : -1;
  }
  // tokens whose pair count is not K: thread m looks after token m
  if (e < M && pairs != K) {
    atomicAdd(violations, 1);
    for (int kk = pairs; kk < K; ++kk) inv[(int64_t)e * K + kk] = -1;
  }
}

// A tile table for another tile height from the prefix sums of a finished index build.
__global__ __launch_bounds__(1024) void tile_table_kernel(const int32_t* __restrict__ cumsums, int N,
                                                          int64_t msum_cap, int tile_rows,
                                                          int32_t* __restrict__ table) {
  __shared__ int32_t s_first[kMaxExperts];
  __shared__ int32_t s_tiles;
  const int t = threadIdx.x, lane = t & 63;
  if (t < 64) {
    int run_tiles = 0;
    for (int i0 = 0; i0 < N; i0 += 64) {
      const int i = i0 + lane;
      const int v = i < N ? cumsums[i + 1] - cumsums[i] : 0;
      const int nt = (v + tile_rows - 1) / tile_rows;
      const int inct = wave_inclusive_scan(nt, lane);
      if (i < N) s_first[i] = run_tiles + inct - nt;
      run_tiles += __shfl(inct, 63);
    }
    if (lane == 0) {
      // an index build that found more pairs than rows emptied its table: so does this one
      const int ntiles = (int64_t)cumsums[N] > msum_cap ? 0 : run_tiles;
      s_tiles = ntiles;
      table[0] = ntiles;
      table[1] = tile_rows;
      table[2] = 0;
      table[3] = 0;
    }
  }
  __syncthreads();
  if (s_tiles == 0) return;
  for (int i = t; i < N; i += 1024) {
    const int c = cumsums[i], v = cumsums[i + 1] - c;
    const int nt = (v + tile_rows - 1) / tile_rows;
    const int first = s_first[i];
    for (int k = 0; k < nt; ++k) {
      int32_t* e = table + kTileHeader + 4 * (first + k);
      e[0] = i;
      e[1] = first;
      e[2] = c;
      e[3] = v;
    }
  }
}

}  // namespace
}  // namespace momoe

using namespace momoe;

// The GEMMs deal an expert's 32-row fragment rows to its ceil(rows / tile_rows) tiles: with a tile
// height below 32, or one that is not a whole number of fragment rows, there would be more tiles
// than fragment rows (tiles without rows, addressed past the expert's end) or tiles taller than
// the height the table promises.  No GEMM takes tiles above MOMOE_TILE_ROWS.
static bool tile_height_ok(int tile_rows) {
  return tile_rows >= 32 && tile_rows <= MOMOE_TILE_ROWS && tile_rows % 32 == 0;
}

extern "C" int momoe_tile_table_build(const int32_t* cumsums_N1, int64_t N, int64_t Msum,
                                      int tile_rows, int32_t* tile_table, void* stream) {
  if (!cumsums_N1 || !tile_table || N <= 0 || Msum <= 0 || tile_rows <= 0) return MOMOE_ERR_BAD_ARG;
  if (N > kMaxExperts || Msum >= (1ll << 31) || !tile_height_ok(tile_rows)) return MOMOE_ERR_UNSUPPORTED;
  tile_table_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(cumsums_N1, (int)N, Msum, tile_rows, tile_table);
  return launch_status();
}

extern "C" int64_t momoe_tile_table_ints(int64_t M, int64_t N, int64_t K, int tile_rows) {
  if (M < 0 || N < 0 || K < 0 || tile_rows < 0) return -1;
  // 0 = the library chooses between two heights: room for the shorter one
  return kTileHeader + 4 * max_row_tiles(M * K, N, tile_rows > 0 ? tile_rows : MOMOE_RECOMPUTE_TILE_ROWS);
}

extern "C" int64_t momoe_index_workspace_bytes(int64_t M, int64_t N) {
  if (M < 0 || N < 0) return -1;
  const int64_t NC = cdiv64(M, kPanelTokens), NG = cdiv64(N, kPanelExperts);
  return (N * NC + NG * M) * (int64_t)sizeof(int32_t) + 256;
}

extern "C" int momoe_index_build(const int32_t* mask_NM, int64_t stride_n, int64_t stride_m,
                                 int64_t M, int64_t N, int64_t K, int64_t* sizes_N,
                                 int32_t* cumsums_N1, int32_t* idx_Msum, int32_t* which_Msum,
                                 int32_t* inv_MK, int32_t* tile_table, int tile_rows,
                                 int32_t* recompute_table, void* workspace,
                                 int64_t workspace_bytes, int32_t* violations, void* stream) {
  if (!mask_NM || !sizes_N || !cumsums_N1 || !idx_Msum || !which_Msum || !inv_MK || !tile_table ||
      !workspace || !violations)
    return MOMOE_ERR_BAD_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || tile_rows < 0) return MOMOE_ERR_BAD_ARG;
  if (N > kMaxExperts || M * K >= (1ll << 31) || M >= (1ll << 30)) return MOMOE_ERR_UNSUPPORTED;
  if (tile_rows != 0 && !tile_height_ok(tile_rows)) return MOMOE_ERR_UNSUPPORTED;
  // the second table goes with the library's own choice of the height
  if (recompute_table != nullptr && tile_rows != 0) return MOMOE_ERR_BAD_ARG;
  if (workspace_bytes < momoe_index_workspace_bytes(M, N)) return MOMOE_ERR_BAD_ARG;
  const int NC = (int)cdiv64(M, kPanelTokens), NG = (int)cdiv64(N, kPanelExperts);
  if (NG > 65535) return MOMOE_ERR_UNSUPPORTED;
  int32_t* part = (int32_t*)workspace;
  int32_t* tokcnt = part + N * NC;
  hipStream_t st = (hipStream_t)stream;
  if (M <= kTinyTokens && N <= kPanelTokens) {
    auto kernel = M <= 16 ? index_tiny_kernel<1> : M <= 32 ? index_tiny_kernel<2>
                : M <= 48 ? index_tiny_kernel<3> : index_tiny_kernel<4>;
    const bool rows_of_int4 = stride_m == 1 && stride_n % 4 == 0 && M % 4 == 0 && ((uintptr_t)mask_NM & 15) == 0;
    kernel<<<1, kPanelTokens, 0, st>>>(mask_NM, stride_n, stride_m, (int)M, (int)N, (int)K, sizes_N,
                                       cumsums_N1, idx_Msum, which_Msum, inv_MK, tile_table,
                                       tile_rows, recompute_table, violations, rows_of_int4);
    return launch_status();
  }
  if (NC == 1 && N <= kSmallMaxExperts) {
    auto kernel = N <= 128 ? index_small_kernel<8> : index_small_kernel<kSmallMaxGroups>;
    kernel<<<1, kPanelTokens, 0, st>>>(mask_NM, stride_n, stride_m, (int)M, (int)N, (int)K, sizes_N,
                                       cumsums_N1, idx_Msum, which_Msum, inv_MK, tile_table,
                                       tile_rows, recompute_table, violations);
    return launch_status();
  }
  dim3 grid(NC, NG);
  index_count_kernel<<<grid, kPanelTokens, 0, st>>>(mask_NM, stride_n, stride_m, (int)M, (int)N,
                                                    NC, part, tokcnt);
  index_scan_kernel<<<1, 1024, 0, st>>>(part, (int)N, NC, M * K, sizes_N, cumsums_N1, tile_table,
                                        tile_rows, recompute_table, violations, idx_Msum,
                                        which_Msum);
  index_scatter_kernel<<<grid, kPanelTokens, 0, st>>>(mask_NM, stride_n, stride_m, (int)M, (int)N,
                                                      (int)K, NC, part, tokcnt, cumsums_N1,
                                                      idx_Msum, which_Msum, inv_MK, violations);
  return launch_status();
}

// ---- the same without a caller-provided workspace ------------------------------------------
// The panel counts live in a fixed array in device memory that is part of the library's code
// object: every GPU the library runs on holds its own copy, at its own address, until the
// process ends.  In host code the array's NAME is only a handle for the runtime, not a device
// address: the address is looked up once per device and kept; kernels and every other use of
// the array's memory take that pointer.
namespace {
constexpr int64_t kStaticScratchBytes = MOMOE_INDEX_STATIC_SCRATCH_BYTES;
__attribute__((used)) static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on device d, once looked up

int scratch_of_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MOMOE_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return MOMOE_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MOMOE_OK;
}
}  // namespace

extern "C" int momoe_index_build_static(const int32_t* mask_NM, int64_t stride_n, int64_t stride_m,
                                        int64_t M, int64_t N, int64_t K, int64_t* sizes_N,
                                        int32_t* cumsums_N1, int32_t* idx_Msum,
                                        int32_t* which_Msum, int32_t* inv_MK, int32_t* tile_table,
                                        int tile_rows, int32_t* recompute_table,
                                        int32_t* violations, void* stream) {
  if (M <= 0 || N <= 0) return MOMOE_ERR_BAD_ARG;
  // sizes beyond the fixed array are refused, never truncated
  if (momoe_index_workspace_bytes(M, N) > kStaticScratchBytes) return MOMOE_ERR_UNSUPPORTED;
  void* ws = nullptr;
  const int st = scratch_of_current_device(&ws);
  if (st != MOMOE_OK) return st;
  // Every word of the array that the scatter pass reads was written by the count pass of the
  // same call, so nothing has to be cleared between calls.
  return momoe_index_build(mask_NM, stride_n, stride_m, M, N, K, sizes_N, cumsums_N1, idx_Msum,
                           which_Msum, inv_MK, tile_table, tile_rows, recompute_table, ws,
                           kStaticScratchBytes, violations, stream);
}
