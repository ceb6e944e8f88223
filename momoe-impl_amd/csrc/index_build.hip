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

__device__ __forceinline__ uint32_t load_panel_bits(const int32_t* __restrict__ mask, int64_t sn,
                                                    int64_t sm, int M, int N, int g, int m) {
  uint32_t bits = 0;
#pragma unroll
  for (int e = 0; e < kPanelExperts; ++e) {
    const int i = g * kPanelExperts + e;
    int32_t v = 0;
    if (i < N && m < M) v = mask[(int64_t)i * sn + (int64_t)m * sm];
    bits |= (v != 0 ? 1u : 0u) << e;
  }
  return bits;
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

__global__ __launch_bounds__(1024) void index_scan_kernel(
    int32_t* __restrict__ part, int N, int NC, int64_t msum_cap,
    int64_t* __restrict__ sizes, int32_t* __restrict__ cumsums,
    int32_t* __restrict__ table, int tile_rows, int32_t* __restrict__ violations,
    int32_t* __restrict__ idx, int32_t* __restrict__ which) {
  __shared__ int32_t s_size[kMaxExperts];
  __shared__ int32_t s_cum[kMaxExperts];
  __shared__ int32_t s_first[kMaxExperts];
  __shared__ int32_t s_total[2];
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
  if (s_total[0] == 0) return;
  for (int i = t; i < N; i += 1024) {
    const int v = s_size[i];
    const int nt = (v + tile_rows - 1) / tile_rows;
    const int first = s_first[i];
    for (int k = 0; k < nt; ++k) {
      int32_t* e = table + kTileHeader + 4 * (first + k);
      e[0] = i;
      e[1] = first;
      e[2] = s_cum[i];
      e[3] = v;
    }
  }
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
        if (k < K) inv[(int64_t)m * K + k] = (int32_t)row;
      }
      ++k;
    }
  }
  if (m < M && g == gridDim.y - 1 && k != K) {
    atomicAdd(violations, 1);
    // slots the token does not fill: -1 = "no row" (momoe_combine skips them)
    for (int kk = k; kk < K; ++kk) inv[(int64_t)m * K + kk] = -1;
  }
}

}  // namespace
}  // namespace momoe

using namespace momoe;

extern "C" int64_t momoe_tile_table_ints(int64_t M, int64_t N, int64_t K, int tile_rows) {
  if (M < 0 || N < 0 || K < 0 || tile_rows <= 0) return -1;
  return kTileHeader + 4 * max_row_tiles(M * K, N, tile_rows);
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
                                 void* workspace, int64_t workspace_bytes, int32_t* violations,
                                 void* stream) {
  if (!mask_NM || !sizes_N || !cumsums_N1 || !idx_Msum || !which_Msum || !inv_MK || !tile_table ||
      !workspace || !violations)
    return MOMOE_ERR_BAD_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || tile_rows <= 0) return MOMOE_ERR_BAD_ARG;
  if (N > kMaxExperts || M * K >= (1ll << 31) || M >= (1ll << 30)) return MOMOE_ERR_UNSUPPORTED;
  if (workspace_bytes < momoe_index_workspace_bytes(M, N)) return MOMOE_ERR_BAD_ARG;
  const int NC = (int)cdiv64(M, kPanelTokens), NG = (int)cdiv64(N, kPanelExperts);
  if (NG > 65535) return MOMOE_ERR_UNSUPPORTED;
  int32_t* part = (int32_t*)workspace;
  int32_t* tokcnt = part + N * NC;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(NC, NG);
  index_count_kernel<<<grid, kPanelTokens, 0, st>>>(mask_NM, stride_n, stride_m, (int)M, (int)N,
                                                    NC, part, tokcnt);
  index_scan_kernel<<<1, 1024, 0, st>>>(part, (int)N, NC, M * K, sizes_N, cumsums_N1, tile_table,
                                        tile_rows, violations, idx_Msum, which_Msum);
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
                                        int tile_rows, int32_t* violations, void* stream) {
  if (M <= 0 || N <= 0) return MOMOE_ERR_BAD_ARG;
  // sizes beyond the fixed array are refused, never truncated
  if (momoe_index_workspace_bytes(M, N) > kStaticScratchBytes) return MOMOE_ERR_UNSUPPORTED;
  void* ws = nullptr;
  const int st = scratch_of_current_device(&ws);
  if (st != MOMOE_OK) return st;
  // Every word of the array that the scatter pass reads was written by the count pass of the
  // same call, so nothing has to be cleared between calls.
  return momoe_index_build(mask_NM, stride_n, stride_m, M, N, K, sizes_N, cumsums_N1, idx_Msum,
                           which_Msum, inv_MK, tile_table, tile_rows, ws, kStaticScratchBytes,
                           violations, stream);
}
