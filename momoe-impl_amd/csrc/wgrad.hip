// Weight-gradient grouped GEMM: GW[i] = A_i^T . B_i, contracting over the sorted
// rows of expert i.  Both operands are stored [row][feature], i.e. k-strided, so
// both go through the LDS transpose read.  Rows may be gathered through an index
// (x and G_y are never materialised in sorted order); the k-values past the expert's
// last row are zeroed in registers.
#include "gemm_tile.hpp"

namespace momoe {
namespace {

constexpr int BX = 256;  // output rows per tile (features of A)
constexpr int BY = 256;  // output columns per tile (features of B)
constexpr int FM = 4, FN = 2;  // 2x4 waves, each 128 x 64
using Ring = StageRing<TGatherDma, TGatherDma>;
constexpr size_t kWgradLds = Ring::BYTES + kEpilogueLds;  // stage ring + per-wave store staging

struct WgradArgs {
  const bf16* a;
  int64_t lda;
  const int32_t* ga;
  const bf16* b;
  int64_t ldb;
  const int32_t* gb;
  const int32_t* cumsums;
  bf16* gw;
  int N, X, Y;
  int tiles_x, tiles_y;
};

struct WTile {
  int expert, x0, y0;
  bool valid;
};

constexpr int kEpilogueCost = 4;  // a tile's epilogue, in units of one k-stage of its main loop

// Persistent workgroups.  id%8 is the XCD a workgroup lands on.  Tiles are numbered expert
// by expert and cut into 8 contiguous runs of equal estimated cost (a tile costs its expert's
// k-stages plus the epilogue), one per XCD: an expert's rows are then fetched from HBM by one
// L2 (two for an expert that straddles a cut) and re-read from there by all of its tiles, and
// an expert that holds far more rows than the others does not hold up one XCD.
__global__ __launch_bounds__(kThreads, 2) void wgrad_kernel(WgradArgs p) {
  Ring ring(dyn_lds());
  const int tpe = p.tiles_x * p.tiles_y;
  const int xcd = blockIdx.x & 7, stride = gridDim.x >> 3;

  // pre[e] = cost of all tiles of the experts before e (exclusive prefix sum), in the stage ring
  int64_t* pre = (int64_t*)dyn_lds();
  int64_t* wave_tot = pre + p.N + 1;
  {
    const int per = (p.N + kThreads - 1) / kThreads;  // experts per thread, contiguous
    const int e0 = min((int)threadIdx.x * per, p.N), e1 = min(e0 + per, p.N);
    int64_t mine = 0;
    for (int e = e0; e < e1; ++e)
      mine += (int64_t)tpe * ((p.cumsums[e + 1] - p.cumsums[e] + kBK - 1) / kBK + kEpilogueCost);
    int64_t incl = mine;  // inclusive scan over the wave, then over the waves
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int64_t v = __shfl_up(incl, o);
      if ((int)(threadIdx.x & 63) >= o) incl += v;
    }
    if ((threadIdx.x & 63) == 63) wave_tot[threadIdx.x >> 6] = incl;
    __syncthreads();
    int64_t base = 0;
    for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) base += wave_tot[w];
    int64_t run = base + incl - mine;
    for (int e = e0; e < e1; ++e) {
      pre[e] = run;
      run += (int64_t)tpe * ((p.cumsums[e + 1] - p.cumsums[e] + kBK - 1) / kBK + kEpilogueCost);
    }
    if (threadIdx.x == kThreads - 1) pre[p.N] = run;
    __syncthreads();
  }
  // first tile whose cost interval starts at or after `c`
  auto tile_at = [&](int64_t c) -> int64_t {
    if (c >= pre[p.N]) return (int64_t)p.N * tpe;
    int lo = 0, hi = p.N;  // pre[lo] <= c < pre[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (pre[mid] <= c) lo = mid; else hi = mid;
    }
    const int64_t each = (pre[lo + 1] - pre[lo]) / tpe;
    return (int64_t)lo * tpe + (c - pre[lo] + each - 1) / each;
  };
  const int64_t total_cost = pre[p.N];
  const int64_t g_begin = tile_at(total_cost * xcd / 8), g_end = tile_at(total_cost * (xcd + 1) / 8);
  __syncthreads();  // the ring is handed to the transfers
  int64_t pos = g_begin + (blockIdx.x >> 3);
  auto next_tile = [&]() {
    WTile t;
    t.valid = pos < g_end;
    if (t.valid) {
      const int expert = (int)(pos / tpe), q = (int)(pos % tpe);
      pos += stride;
      t.expert = expert;
      t.x0 = (q / p.tiles_y) * BX;
      t.y0 = (q % p.tiles_y) * BY;
    }
    return t;
  };
  TGatherDma A, B;
  int cur_expert = -1, rb = 0, re = 0;
  // the rows of an expert (and the ids of the first of them) are looked up when the
  // workgroup moves on to a new expert; every tile of the expert then reuses them
  auto start = [&](const WTile& t) {
    if (t.expert != cur_expert) {
      cur_expert = t.expert;
      rb = load_uniform(p.cumsums + t.expert);
      re = load_uniform(p.cumsums + t.expert + 1);
      if (re > rb) {
        A.set_rows(p.ga, p.lda, rb, re);
        B.set_rows(p.gb, p.ldb, rb, re);
      }
    }
    if (re <= rb) return;  // expert without rows: nothing to load, zeros are stored
    A.set_cols(p.a, t.x0, p.X);
    B.set_cols(p.b, t.y0, p.Y);
    gemm_issue_first(A, B, ring, (re - rb + kBK - 1) / kBK);
  };
  const int wave = threadIdx.x >> 6, wm = wave >> 2, wn = wave & 3;
  const int m_org[FM] = {wm * 128, wm * 128 + 32, wm * 128 + 64, wm * 128 + 96};
  const int n_org[FN] = {wn * 64, wn * 64 + 32};
  RowStager<2> stager(dyn_lds() + kStages * Ring::STAGE);

  WTile tc = next_tile();
  if (!tc.valid) return;
  start(tc);
  while (true) {
    f32x16 acc[FN][FM];
    zero_acc<FM, FN>(acc);
    const int ktiles = (re - rb + kBK - 1) / kBK;  // rows of tc's expert (start(tc) ran last)
    const int ktail = re - rb - (ktiles - 1) * kBK;
    const WTile nx = next_tile();
    if (ktiles > 0)
      gemm_mainloop<TGatherDma, TGatherDma, FM, FN, FM>(A, B, acc, ktiles, ring, m_org, n_org, [] {}, ktail);
    if (nx.valid) start(nx);

    bf16* out = p.gw + (int64_t)tc.expert * p.X * p.Y;
    const int y0 = tc.y0 + wn * 64;  // first output column of this wave
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd)
          stager.put(f, qd, pack_bf16x4(acc[f][i][4 * qd], acc[f][i][4 * qd + 1],
                                        acc[f][i][4 * qd + 2], acc[f][i][4 * qd + 3]));
      stager.flush<true>([&](int row, int col) -> bf16* {
        const int x = tc.x0 + m_org[i] + row;
        if (x >= p.X || y0 + col >= p.Y) return nullptr;
        return out + (int64_t)x * p.Y + y0 + col;
      });
    }
    if (!nx.valid) break;
    tc = nx;
  }
}

}  // namespace
}  // namespace momoe

using namespace momoe;

extern "C" int momoe_wgrad(const void* A_rows, int64_t lda, const int32_t* a_gather,
                           const void* B_rows, int64_t ldb, const int32_t* b_gather,
                           const int32_t* cumsums_N1, void* GW_NXY, int64_t M, int64_t N,
                           int64_t X, int64_t Y, int64_t Msum, void* stream) {
  if (!A_rows || !B_rows || !cumsums_N1 || !GW_NXY) return MOMOE_ERR_BAD_ARG;
  if (M <= 0 || N <= 0 || X <= 0 || Y <= 0 || Msum <= 0 || lda < X || ldb < Y)
    return MOMOE_ERR_BAD_ARG;
  if (X % 8 != 0 || Y % 8 != 0 || lda % 8 != 0 || ldb % 8 != 0) return MOMOE_ERR_UNSUPPORTED;
  if (((uintptr_t)A_rows & 15) || ((uintptr_t)B_rows & 15) || ((uintptr_t)GW_NXY & 7))
    return MOMOE_ERR_BAD_ARG;
  if (Msum >= (1ll << 31) || X > (1 << 20) || Y > (1 << 20)) return MOMOE_ERR_UNSUPPORTED;
  // rows are addressed with 32-bit byte offsets from the matrix base (gathered: M rows) or from
  // the expert's first row (an expert holds a token at most once: at most M rows)
  if (M * lda * 2 >= (1ll << 32) || M * ldb * 2 >= (1ll << 32)) return MOMOE_ERR_UNSUPPORTED;
  const int tiles_x = (int)cdiv64(X, BX), tiles_y = (int)cdiv64(Y, BY);
  // the per-expert cost prefix sums live in LDS while the tiles are dealt out
  if ((int64_t)tiles_x * tiles_y >= (1ll << 31) || N > 8192) return MOMOE_ERR_UNSUPPORTED;
  WgradArgs a{(const bf16*)A_rows, lda, a_gather, (const bf16*)B_rows, ldb, b_gather, cumsums_N1,
              (bf16*)GW_NXY, (int)N, (int)X, (int)Y, tiles_x, tiles_y};
  static std::once_flag once;
  allow_lds(wgrad_kernel, kWgradLds, once);
  wgrad_kernel<<<persistent_grid(), kThreads, kWgradLds, (hipStream_t)stream>>>(a);
  return launch_status();
}
