// Weight-gradient grouped GEMM: GW[i] = A_i^T . B_i, contracting over the sorted
// rows of expert i.  An operand is handed over in one of two layouts:
//   rows        [row][feature] (optionally gathered through an index: x and G_y are never
//               materialised in sorted order).  The contraction index is the slow one, so its
//               fragments come through the LDS transpose read, at half the rate of a plain read.
//   transposed  [padded sorted row / 32][feature][32]: the producing kernel wrote the matrix in
//               groups of 32 rows, feature-major inside a group (hs), each expert's rows starting
//               at a multiple of 32 and zero-filled up to the next multiple of 32.  The
//               contraction index is the fast one: plain 16-byte fragment reads, and a stage is
//               one contiguous 16 KiB block in memory.
// Per wave and k-step the 4-fragment side of the 128 x 64 wave tile reads twice the LDS bytes of
// the 2-fragment side, so the transposed operand is given the 4 fragments: it is the M side
// (FM=4, FN=2) when A is transposed and the N side (FM=2, FN=4) when B is.
// The k-values past the expert's last row are zeroed in registers on the M side.
#include <algorithm>

#include "gemm_tile.hpp"

namespace momoe {
namespace {

constexpr int BX = 256;  // output rows per tile (features of A)
constexpr int BY = 256;  // output columns per tile (features of B)
constexpr int kStages = 4;  // ring depth
constexpr int kRingBytes = kStages * 2 * TLayout::LDS_ELEMS * 2;  // every operand kind: 16 KiB per stage
constexpr size_t kWgradLds = kRingBytes + kEpilogueLds;  // stage ring + per-wave store staging
constexpr int kMaxWgradExperts = 4096;  // 20 bytes of prefix sums per expert fit the stage ring
constexpr int kMaxWorkgroups = 256;       // the workspace query assumes no more persistent workgroups
constexpr int kSplitsPerWorkgroup = 8;  // large experts are cut into pieces of 1/8 .. 1/4 of a
                                        // workgroup's share of the launch
static_assert(BX * BY * 4 == MOMOE_WGRAD_PARTIAL_BYTES, "size of one fp32 partial tile");
static_assert((size_t)(kMaxWgradExperts + 1) * 20 + 512 <= kRingBytes, "prefix sums overlay the ring");

// "rows" operand of a work item: the gathered / sorted rows [rb, re)
struct RowsOperand : TGatherDmaT<true, kStages - 1> {
  __device__ __forceinline__ void begin_piece(const int32_t* gather_, int64_t ld_, int rb, int re, int) {
    set_rows(gather_, ld_, rb, re);
  }
};
// "k-blocked" operand: sorted rows (no gather) of a matrix stored in blocks of 32 features,
// feature f of row r at mat[((f / 32) * ld + r) * 32 + f % 32], ld = rows of the matrix (gz, as
// the SwiGLU backward writes it for dL/dx).  Rows are the contraction index, as in the row layout,
// and go through the same transposing LDS reads; the 32 rows x 32 features of a block are 2 KiB
// of consecutive memory.
struct BlockedRowsOperand : TGatherDmaT<false, kStages - 1> {
  int64_t nrows;
  __device__ __forceinline__ void begin_piece(const int32_t*, int64_t ld_, int rb, int re, int) {
    nrows = ld_;
    set_rows(nullptr, 32, rb, re);  // row pitch: 32 elements
  }
  // features [col0, col0+256) (col0 a multiple of 256); features >= ncols are clamped to col0
  __device__ __forceinline__ void set_cols(const bf16* mat_, int col0, int ncols) {
    mat = mat_ + ((int64_t)(col0 >> 5) * nrows + row_begin) * 32;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      int krow, c;
      L::lane_piece(j, krow, c);
      const int cc = col0 + c < ncols ? c : 0;
      colb[j] = (uint32_t)(((int64_t)(cc >> 5) * nrows * 32 + (cc & 31)) * 2);
    }
  }
};

// "transposed" operand: groups of 32 padded sorted rows, feature-major inside a group: feature f
// of padded sorted row p at mat[(p / 32) * ld * 32 + f * 32 + p % 32], ld >= number of features.
// The 256 features x 32 rows of one stage are 16 KiB of consecutive memory.
struct TransposedOperand {
  using R = RDma<256>;
  static constexpr int NCH = R::NCH;
  static constexpr int LDS_ELEMS = R::LDS_ELEMS;
  static_assert(LDS_ELEMS == TLayout::LDS_ELEMS, "same stage size as the other operand kind");
  R r;
  int64_t gstride;  // elements between consecutive 32-row groups
  int g0;           // group of the first row of the piece
  __device__ __forceinline__ void begin_piece(const int32_t*, int64_t ld_, int, int, int prow) {
    gstride = ld_ * 32;
    g0 = prow >> 5;
  }
  // features [f0, f0+256) of the matrix; features >= nfeat are clamped to the last one
  __device__ __forceinline__ void set_cols(const bf16* mat, int f0, int nfeat) {
    r.init(mat + (int64_t)g0 * gstride + (int64_t)f0 * 32,
           [&](int row, int) { return (uint32_t)min(row, nfeat - 1 - f0) * 64u; });
  }
  __device__ __forceinline__ void issue(int kt, uint32_t stage) {
    const int w = wave_id();
    const bf16* b = r.base + (int64_t)kt * gstride;
#pragma unroll
    for (int j = 0; j < NCH; ++j) dma16(b, r.off[j], stage + (j * kWaves + w) * (kChunkElems * 2));
  }
  template <int S>
  __device__ __forceinline__ void issue_head(uint32_t stage) { issue(S, stage); }
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int c0, int kk) { return R::frag(stage, c0, kk); }
};

struct WgradArgs {
  const bf16* a;
  int64_t lda;
  const int32_t* ga;
  const bf16* b;
  int64_t ldb;
  const int32_t* gb;
  const int32_t* cumsums;
  bf16* gw;
  float* ws;      // fp32 partial tiles of the experts that are cut along their rows
  int kc;         // experts of at least 2*kc k-stages are cut into pieces of kc .. 2*kc stages
  int N, X, Y;
  int tiles_x, tiles_y;
  int msum;       // rows of the sorted matrices: row counts are clamped to it
  unsigned long long* clk;
};

struct WTile {
  int expert, x0, y0;
  int rb, re;  // sorted rows this work item contracts over
  int prow;    // padded position of row rb (transposed operands)
  int slot;    // partial tile to write, or -1: the item covers the whole expert and stores bf16
  bool valid;
};

// How the 8 waves share the 256 x 256 output tile: FM x FN fragments of 32 x 32 per wave.
template <int FM, int FN>
struct WaveTile {
  static_assert(FM * FN == 8 && (FM == 4 || FM == 2), "128 x 64 or 64 x 128 per wave");
  static constexpr int WAVES_N = 256 / (32 * FN);  // waves side by side
  int m_org[FM], n_org[FN];
  __device__ __forceinline__ WaveTile() {
    const int wave = wave_id(), wm = wave / WAVES_N, wn = wave % WAVES_N;
#pragma unroll
    for (int i = 0; i < FM; ++i) m_org[i] = wm * (32 * FM) + 32 * i;
#pragma unroll
    for (int j = 0; j < FN; ++j) n_org[j] = wn * (32 * FN) + 32 * j;
  }
};

constexpr int kEpilogueCost = 4;  // a tile's epilogue, in units of one k-stage of its main loop
constexpr int kMinChunk = 64;     // an expert is never cut into pieces of fewer k-stages

// How one expert's rows are dealt out: `splits` equal pieces of `chunk` k-stages (the last
// may be shorter).  An expert is cut once it holds at least 2*kc stages, so a piece has
// between kc and 2*kc stages.
struct ExpertPlan {
  int ks, splits, chunk;
};
__device__ __forceinline__ ExpertPlan plan_expert(int rows, int kc) {
  ExpertPlan e;
  e.ks = (rows + kBK - 1) / kBK;
  e.splits = max(1, e.ks / kc);
  e.chunk = (e.ks + e.splits - 1) / e.splits;
  return e;
}

// Prefix sums over the experts, kept in LDS while the work is dealt out (they overlay the
// stage ring).  A work item is one output tile of one piece of one expert; inside an expert
// the items run piece by piece, tile by tile.
struct Plan {
  int64_t* cost;    // [N+1] estimated cost of the items of the experts before e
  int32_t* items;   // [N+1] items of the experts before e
  int32_t* slots;   // [N+1] partial tiles of the experts before e (cut experts only)
  int32_t* ctiles;  // [N+1] output tiles of the cut experts before e
  int kc;
};

__device__ __forceinline__ Plan build_plan(const WgradArgs& p, int tpe) {
  Plan pl;
  pl.cost = (int64_t*)dyn_lds();
  pl.items = (int32_t*)(pl.cost + p.N + 1);
  pl.slots = pl.items + p.N + 1;
  pl.ctiles = pl.slots + p.N + 1;
  int64_t* wt = (int64_t*)(((uintptr_t)(pl.ctiles + p.N + 1) + 7) & ~(uintptr_t)7);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int per = (p.N + kThreads - 1) / kThreads;  // experts per thread, contiguous
  const int e0 = min((int)threadIdx.x * per, p.N), e1 = min(e0 + per, p.N);

  pl.kc = p.kc;

  // exclusive scans of cost / items / slots / cut tiles over the experts
  int64_t c = 0;
  int32_t n = 0, sl = 0, ct = 0;
  for (int e = e0; e < e1; ++e) {
    const ExpertPlan ep = plan_expert(min(p.cumsums[e + 1], p.msum) - min(p.cumsums[e], p.msum), pl.kc);
    const int ne = tpe * ep.splits;
    c += (int64_t)ne * (ep.chunk + kEpilogueCost);
    n += ne;
    if (ep.splits > 1) sl += ne, ct += tpe;
  }
  int64_t ic = c;
  int32_t in = n, isl = sl, ict = ct;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int64_t vc = __shfl_up(ic, o);
    const int32_t vn = __shfl_up(in, o), vs = __shfl_up(isl, o), vt = __shfl_up(ict, o);
    if (lane >= o) ic += vc, in += vn, isl += vs, ict += vt;
  }
  if (lane == 63) {  // per wave: cost, items, slots, cut tiles
    wt[4 * wave] = ic;
    wt[4 * wave + 1] = in;
    wt[4 * wave + 2] = isl;
    wt[4 * wave + 3] = ict;
  }
  __syncthreads();
  int64_t bc = 0;
  int32_t bn = 0, bs = 0, bt = 0;
  for (int w = 0; w < wave; ++w) {
    bc += wt[4 * w];
    bn += (int32_t)wt[4 * w + 1];
    bs += (int32_t)wt[4 * w + 2];
    bt += (int32_t)wt[4 * w + 3];
  }
  bc += ic - c, bn += in - n, bs += isl - sl, bt += ict - ct;
  for (int e = e0; e < e1; ++e) {
    pl.cost[e] = bc, pl.items[e] = bn, pl.slots[e] = bs, pl.ctiles[e] = bt;
    const ExpertPlan ep = plan_expert(min(p.cumsums[e + 1], p.msum) - min(p.cumsums[e], p.msum), pl.kc);
    const int ne = tpe * ep.splits;
    bc += (int64_t)ne * (ep.chunk + kEpilogueCost);
    bn += ne;
    if (ep.splits > 1) bs += ne, bt += tpe;
  }
  if (threadIdx.x == kThreads - 1)
    pl.cost[p.N] = bc, pl.items[p.N] = bn, pl.slots[p.N] = bs, pl.ctiles[p.N] = bt;
  __syncthreads();
  return pl;
}

// The same when no expert is cut: only the cost prefix sums are needed, an expert's items
// are its tpe tiles.
__device__ __forceinline__ Plan build_cost_plan(const WgradArgs& p, int tpe) {
  Plan pl;
  pl.cost = (int64_t*)dyn_lds();
  pl.items = pl.slots = pl.ctiles = nullptr;
  pl.kc = 0x7fffffff;
  int64_t* wave_tot = pl.cost + p.N + 1;
  const int per = (p.N + kThreads - 1) / kThreads;  // experts per thread, contiguous
  const int e0 = min((int)threadIdx.x * per, p.N), e1 = min(e0 + per, p.N);
  auto cost_of = [&](int e) {
    const int rows = min(p.cumsums[e + 1], p.msum) - min(p.cumsums[e], p.msum);
    return (int64_t)tpe * ((rows + kBK - 1) / kBK + kEpilogueCost);
  };
  int64_t mine = 0;
  for (int e = e0; e < e1; ++e) mine += cost_of(e);
  int64_t incl = mine;  // inclusive scan over the wave, then over the waves
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int64_t v = __shfl_up(incl, o);
    if ((int)(threadIdx.x & 63) >= o) incl += v;
  }
  if ((threadIdx.x & 63) == 63) wave_tot[threadIdx.x >> 6] = incl;
  __syncthreads();
  int64_t run = incl - mine;
  for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) run += wave_tot[w];
  for (int e = e0; e < e1; ++e) {
    pl.cost[e] = run;
    run += cost_of(e);
  }
  if (threadIdx.x == kThreads - 1) pl.cost[p.N] = run;
  __syncthreads();
  return pl;
}

// bf16 store of one output tile from the accumulators (non-temporal: a weight gradient is
// not read again by this kernel); two fragments (64 columns) go through the staging area at a time
template <int FM, int FN>
__device__ __forceinline__ void store_gw_tile(const WgradArgs& p, RowStager<2>& stager,
                                              f32x16 (&acc)[FN][FM], int expert, int x0, int y0t,
                                              const WaveTile<FM, FN>& wt) {
  bf16* out = p.gw + (int64_t)expert * p.X * p.Y;
#pragma unroll
  for (int i = 0; i < FM; ++i) {
#pragma unroll
    for (int f0 = 0; f0 < FN; f0 += 2) {
#pragma unroll
      for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd)
          stager.put(f, qd, pack_bf16x4(acc[f0 + f][i][4 * qd], acc[f0 + f][i][4 * qd + 1],
                                        acc[f0 + f][i][4 * qd + 2], acc[f0 + f][i][4 * qd + 3]));
      const int y0 = y0t + wt.n_org[f0];  // first output column of these two fragments
      stager.flush<true>([&](int row, int col) -> bf16* {
        const int x = x0 + wt.m_org[i] + row;
        if (x >= p.X || y0 + col >= p.Y) return nullptr;
        return out + (int64_t)x * p.Y + y0 + col;
      });
    }
  }
}

// values read back from LDS are the same in every lane; tell the compiler so
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// A partial tile is kept in accumulator order: per wave, per fragment, 4 x (64 lanes x 16 B).
template <int FM, int FN>
__device__ __forceinline__ f32x4* partial_piece(float* ws, int slot, int i, int f, int qd) {
  const int wave = wave_id(), lane = threadIdx.x & 63;
  return (f32x4*)(ws + (int64_t)slot * (BX * BY)) +
         ((((wave * FM + i) * FN + f) * 4 + qd) * 64 + lane);
}

// Persistent workgroups.  id%8 is the XCD a workgroup lands on.  Work items are numbered
// expert by expert and cut into 8 contiguous runs of equal estimated cost (an item costs its
// k-stages plus the epilogue), one per XCD, whose workgroups walk the run with a stride: an
// expert's rows are then fetched from HBM by one L2 (two for an expert that straddles a cut)
// and re-read from there by all of its tiles.  An expert with many times the rows of the
// others would make single tiles as long as a workgroup's whole share, so its rows are cut
// into pieces; the pieces of a tile go to the workspace in fp32 and wgrad_reduce_kernel adds
// them up.
// CUT = false is the launch in which no expert can reach the cutting length (the host knows:
// an expert holds at most M rows): the bookkeeping of pieces is compiled out.
// A routing with more pairs than sorted rows (cumsums[N] > Msum) got an empty tile table: the
// GEMMs before this one wrote nothing, so no expert has rows to contract over and every weight
// gradient is zero.  Row counts are clamped to p.msum everywhere: clamp them to nothing.
__device__ __forceinline__ void drop_rows_of_an_overflowed_routing(WgradArgs& p) {
  if (load_uniform(p.cumsums + p.N) > p.msum) p.msum = 0;
}

template <bool CUT, class AOp, class BOp, int FM, int FN>
__global__ __launch_bounds__(kThreads, 2) void wgrad_kernel(WgradArgs p) {
  drop_rows_of_an_overflowed_routing(p);
  using Ring = StageRing<AOp, BOp, kStages>;
  static_assert(Ring::BYTES == kRingBytes, "ring size assumed by the launch");
  const ClockTrace trace(p.clk);
  Ring ring(dyn_lds());
  const int tpe = p.tiles_x * p.tiles_y;
  const int xcd = blockIdx.x & 7, stride = gridDim.x >> 3;
  const Plan pl = CUT ? build_plan(p, tpe) : build_cost_plan(p, tpe);
  const int kc = CUT ? uniform(pl.kc) : 0x7fffffff;
  auto items_before = [&](int e) { return CUT ? pl.items[e] : e * tpe; };

  // first item whose cost interval starts at or after `c`
  auto item_at = [&](int64_t c) -> int {
    if (c >= pl.cost[p.N]) return items_before(p.N);
    int lo = 0, hi = p.N;  // cost[lo] <= c < cost[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (pl.cost[mid] <= c) lo = mid; else hi = mid;
    }
    const int64_t each = (pl.cost[lo + 1] - pl.cost[lo]) / (items_before(lo + 1) - items_before(lo));
    return items_before(lo) + (int)((c - pl.cost[lo] + each - 1) / each);
  };
  const int64_t total_cost = pl.cost[p.N];
  const int g_end = uniform(item_at(total_cost * (xcd + 1) / 8));
  int pos = uniform(item_at(total_cost * xcd / 8)) + (int)(blockIdx.x >> 3);
  // the expert that holds item `pos`; later experts are reached by walking forward
  int ex = 0, ex_first = 0, ex_slot = 0;
  if constexpr (CUT) {
    int lo = 0, hi = p.N;  // items[lo] <= pos < items[hi] (if pos is an item at all)
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (pl.items[mid] <= pos) lo = mid; else hi = mid;
    }
    ex = uniform(lo);
    ex_first = uniform(pl.items[ex]);  // first item of expert ex
    ex_slot = uniform(pl.slots[ex]);   // first partial tile of expert ex
  }
  __syncthreads();  // the ring is handed to the transfers
  int ex_rb = 0, ex_re = 0, ahead = 0;
  ExpertPlan ep = {0, 1, 0};
  if constexpr (CUT) {
    ex_rb = min(load_uniform(p.cumsums + ex), p.msum);
    ex_re = min(load_uniform(p.cumsums + ex + 1), p.msum);
    ep = plan_expert(ex_re - ex_rb, kc);
    // end of the next expert's rows, requested one expert ahead so that moving on does not wait
    ahead = load_uniform(p.cumsums + min(ex + 2, p.N));
  }

  auto next_tile = [&]() {
    WTile t;
    t.valid = pos < g_end;
    if (!t.valid) return t;
    if constexpr (!CUT) {
      const int expert = pos / tpe, q = pos - expert * tpe;
      pos += stride;
      t.expert = expert;
      t.x0 = (q / p.tiles_y) * BX;
      t.y0 = (q % p.tiles_y) * BY;
      t.rb = min(load_uniform(p.cumsums + expert), p.msum);
      t.re = min(load_uniform(p.cumsums + expert + 1), p.msum);
      t.prow = padded_start(t.rb, expert);
      t.slot = -1;
      return t;
    }
    while (pos >= ex_first + tpe * ep.splits && ex + 1 < p.N) {
      ex_first += tpe * ep.splits;
      if (ep.splits > 1) ex_slot += tpe * ep.splits;
      ++ex;
      ex_rb = ex_re;
      ex_re = min(ahead, p.msum);
      ahead = load_uniform(p.cumsums + min(ex + 2, p.N));
      ep = plan_expert(ex_re - ex_rb, kc);
    }
    const int it = pos - ex_first, piece = it / tpe, q = it - piece * tpe;
    pos += stride;
    t.expert = ex;
    t.x0 = (q / p.tiles_y) * BX;
    t.y0 = (q % p.tiles_y) * BY;
    t.rb = min(ex_re, ex_rb + piece * ep.chunk * kBK);
    t.re = min(ex_re, t.rb + ep.chunk * kBK);
    t.prow = padded_start(ex_rb, ex) + (t.rb - ex_rb);
    t.slot = ep.splits > 1 ? ex_slot + it : -1;
    return t;
  };
  AOp A;
  BOp B;
  int cur_rb = -1, cur_re = -1;
  // the rows of a piece (and the ids of the first of them) are looked up when the workgroup
  // moves on to a new piece; every tile of the piece then reuses them
  auto start = [&](const WTile& t) {
    if (t.re <= t.rb) return;  // no rows: nothing to load, zeros are stored
    if (t.rb != cur_rb || t.re != cur_re) {
      cur_rb = t.rb;
      cur_re = t.re;
      A.begin_piece(p.ga, p.lda, t.rb, t.re, t.prow);
      B.begin_piece(p.gb, p.ldb, t.rb, t.re, t.prow);
    }
    A.set_cols(p.a, t.x0, p.X);
    B.set_cols(p.b, t.y0, p.Y);
    gemm_issue_first(A, B, ring, (t.re - t.rb + kBK - 1) / kBK);
  };
  const WaveTile<FM, FN> wt;
  RowStager<2> stager(dyn_lds() + kStages * Ring::STAGE);

  WTile tc = next_tile();
  if (!tc.valid) {
    trace.finish();
    return;
  }
  start(tc);
  while (true) {
    f32x16 acc[FN][FM];
    zero_acc<FM, FN>(acc);
    const int ktiles = (tc.re - tc.rb + kBK - 1) / kBK;
    const int ktail = tc.re - tc.rb - (ktiles - 1) * kBK;
    const WTile nx = next_tile();
    if (ktiles > 0)
      gemm_mainloop<AOp, BOp, kStages, FM, FN, FM>(A, B, acc, ktiles, ring, wt.m_org, wt.n_org, [] {}, ktail);
    if (nx.valid) start(nx);

    if (!CUT || tc.slot < 0) {
      store_gw_tile<FM, FN>(p, stager, acc, tc.expert, tc.x0, tc.y0, wt);
    } else {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int f = 0; f < FN; ++f)
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            f32x4 v = {acc[f][i][4 * qd], acc[f][i][4 * qd + 1], acc[f][i][4 * qd + 2],
                       acc[f][i][4 * qd + 3]};
            *partial_piece<FM, FN>(p.ws, tc.slot, i, f, qd) = v;
          }
    }
    if (!nx.valid) break;
    tc = nx;
  }
  trace.finish();
}

// Adds up the partial tiles of the experts that wgrad_kernel cut into pieces and stores the
// bf16 result; one workgroup per output tile, same register layout as the GEMM.
template <int FM, int FN>
__global__ __launch_bounds__(kThreads) void wgrad_reduce_kernel(WgradArgs p) {
  drop_rows_of_an_overflowed_routing(p);
  const int tpe = p.tiles_x * p.tiles_y;
  const Plan pl = build_plan(p, tpe);
  const int ncut = pl.ctiles[p.N];
  const WaveTile<FM, FN> wt;
  RowStager<2> stager((bf16*)((char*)dyn_lds() + kRingBytes));
  for (int t = blockIdx.x; t < ncut; t += gridDim.x) {
    int lo = 0, hi = p.N;  // ctiles[lo] <= t < ctiles[hi]; the last such lo is the cut expert
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (pl.ctiles[mid] <= t) lo = mid; else hi = mid;
    }
    const int q = t - pl.ctiles[lo];
    const int splits = (pl.slots[lo + 1] - pl.slots[lo]) / tpe;
    f32x16 acc[FN][FM];
    zero_acc<FM, FN>(acc);
    for (int piece = 0; piece < splits; ++piece) {
      const int slot = pl.slots[lo] + piece * tpe + q;
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int f = 0; f < FN; ++f)
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            const f32x4 v = *partial_piece<FM, FN>(p.ws, slot, i, f, qd);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[f][i][4 * qd + r] += v[r];
          }
    }
    store_gw_tile<FM, FN>(p, stager, acc, lo, (q / p.tiles_y) * BX, (q % p.tiles_y) * BY, wt);
  }
}

}  // namespace
}  // namespace momoe

using namespace momoe;

// The most partial tiles a launch can use: kSplitsPerWorkgroup per workgroup, and no more than
// the pieces of kMinChunk k-stages that the rows can be cut into.
extern "C" int64_t momoe_wgrad_workspace_bytes(int64_t N, int64_t X, int64_t Y, int64_t Msum) {
  if (N <= 0 || X <= 0 || Y <= 0 || Msum < 0) return -1;
  const int64_t tpe = cdiv64(X, BX) * cdiv64(Y, BY);
  const int64_t by_rows = tpe * (Msum / kBK + N) / kMinChunk;
  return std::min<int64_t>((int64_t)kSplitsPerWorkgroup * kMaxWorkgroups, by_rows) *
         MOMOE_WGRAD_PARTIAL_BYTES;
}

namespace {
template <class AOp, class BOp, int FM, int FN>
int launch_wgrad(const WgradArgs& a, bool can_cut, int grid, hipStream_t st) {
  static LdsLimit once, once_cut, once_reduce;
  if (!can_cut) {
    if (!allow_lds(wgrad_kernel<false, AOp, BOp, FM, FN>, kWgradLds, once)) return MOMOE_ERR_LAUNCH;
    wgrad_kernel<false, AOp, BOp, FM, FN><<<grid, kThreads, kWgradLds, st>>>(a);
  } else {
    if (!allow_lds(wgrad_kernel<true, AOp, BOp, FM, FN>, kWgradLds, once_cut) ||
        !allow_lds(wgrad_reduce_kernel<FM, FN>, kWgradLds, once_reduce))
      return MOMOE_ERR_LAUNCH;
    wgrad_kernel<true, AOp, BOp, FM, FN><<<grid, kThreads, kWgradLds, st>>>(a);
    wgrad_reduce_kernel<FM, FN><<<grid, kThreads, kWgradLds, st>>>(a);
  }
  return launch_status();
}
}  // namespace

extern "C" int64_t momoe_padded_rows(int64_t Msum, int64_t N) {
  if (Msum < 0 || N < 0) return -1;
  return ((Msum + 31) & ~(int64_t)31) + 32 * N;
}

extern "C" int momoe_wgrad(const void* A, int64_t lda, int a_layout, const int32_t* a_gather,
                           const void* B, int64_t ldb, int b_layout, const int32_t* b_gather,
                           const int32_t* cumsums_N1, void* GW_NXY, int64_t M, int64_t N,
                           int64_t X, int64_t Y, int64_t Msum, void* workspace,
                           int64_t workspace_bytes, void* stream) {
  if (!A || !B || !cumsums_N1 || !GW_NXY) return MOMOE_ERR_BAD_ARG;
  if (M <= 0 || N <= 0 || X <= 0 || Y <= 0 || Msum <= 0) return MOMOE_ERR_BAD_ARG;
  const bool at = a_layout == MOMOE_LAYOUT_TRANSPOSED, bt = b_layout == MOMOE_LAYOUT_TRANSPOSED;
  const bool bk = b_layout == MOMOE_LAYOUT_KBLOCKED;
  if ((!at && a_layout != MOMOE_LAYOUT_ROWS) || (!bt && !bk && b_layout != MOMOE_LAYOUT_ROWS))
    return MOMOE_ERR_BAD_ARG;
  if (at && (bt || bk)) return MOMOE_ERR_UNSUPPORTED;  // one operand at most in a special layout
  // k-blocked B: ldb = rows of the matrix; features in whole blocks; 8 blocks of a tile are
  // addressed with 32-bit byte offsets
  if (bk && (b_gather != nullptr || ldb < Msum || Y % 32 != 0 || 8 * ldb * 64 >= (1ll << 32)))
    return b_gather != nullptr || ldb < Msum ? MOMOE_ERR_BAD_ARG : MOMOE_ERR_UNSUPPORTED;
  const int64_t mpad = momoe_padded_rows(Msum, N);
  if (lda < X || (!bk && ldb < Y) || (at && a_gather != nullptr) || (bt && b_gather != nullptr))
    return MOMOE_ERR_BAD_ARG;
  if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace) || ((uintptr_t)workspace & 15))
    return MOMOE_ERR_BAD_ARG;
  if (X % 8 != 0 || Y % 8 != 0 || lda % 8 != 0 || (!bk && ldb % 8 != 0)) return MOMOE_ERR_UNSUPPORTED;
  if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)GW_NXY & 7))
    return MOMOE_ERR_BAD_ARG;
  if (Msum >= (1ll << 31) || mpad >= (1ll << 31) || X > (1 << 20) || Y > (1 << 20))
    return MOMOE_ERR_UNSUPPORTED;
  // rows are addressed with 32-bit byte offsets from the matrix base (gathered: M rows) or from
  // the first row of an expert's piece (an expert holds a token at most once: at most M rows);
  // a transposed operand needs no such offsets (a stage is one contiguous block)
  if ((!at && M * lda * 2 >= (1ll << 32)) || (!bt && !bk && M * ldb * 2 >= (1ll << 32)))
    return MOMOE_ERR_UNSUPPORTED;
  const int tiles_x = (int)cdiv64(X, BX), tiles_y = (int)cdiv64(Y, BY);
  // the per-expert prefix sums live in LDS while the work is dealt out; work items are
  // counted in 32 bits (every expert has its tiles, the cut ones at most ws_tiles more)
  const int grid = persistent_grid();
  const int64_t ws_tiles = std::min<int64_t>(workspace_bytes / MOMOE_WGRAD_PARTIAL_BYTES,
                                             (int64_t)kSplitsPerWorkgroup * std::min(grid, kMaxWorkgroups));
  if (N > kMaxWgradExperts || (int64_t)tiles_x * tiles_y * N + ws_tiles >= (1ll << 31))
    return MOMOE_ERR_UNSUPPORTED;
  // The launch has at most Msum/kBK + N k-stages per output tile.  With pieces of at least kc
  // stages the cut experts make at most tpe * stages / kc partial tiles: kc is chosen so that
  // they fit the workspace.
  int kc = 0x7fffffff;
  if (ws_tiles > 0) {
    const int64_t stages = (int64_t)tiles_x * tiles_y * (Msum / kBK + N);
    kc = (int)std::min<int64_t>(0x7fffffff, std::max<int64_t>(kMinChunk, cdiv64(stages, ws_tiles)));
  }
  WgradArgs a{(const bf16*)A, lda, a_gather, (const bf16*)B, ldb, b_gather, cumsums_N1,
              (bf16*)GW_NXY, (float*)workspace, kc, (int)N, (int)X, (int)Y, tiles_x, tiles_y,
              (int)Msum, clock_trace_buffer()};
  // an expert holds at most M rows: if that is short of the cutting length, nothing is cut
  const bool can_cut = kc != 0x7fffffff && cdiv64(std::min(M, Msum), kBK) >= 2 * (int64_t)kc;
  hipStream_t st = (hipStream_t)stream;
  if (at) return launch_wgrad<TransposedOperand, RowsOperand, 4, 2>(a, can_cut, grid, st);
  if (bt) return launch_wgrad<RowsOperand, TransposedOperand, 2, 4>(a, can_cut, grid, st);
  if (bk) return launch_wgrad<RowsOperand, BlockedRowsOperand, 4, 2>(a, can_cut, grid, st);
  return launch_wgrad<RowsOperand, RowsOperand, 4, 2>(a, can_cut, grid, st);
}
