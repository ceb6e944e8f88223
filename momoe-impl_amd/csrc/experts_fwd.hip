// Forward of the experts: grouped GEMM x.Wl1 with fused SwiGLU, grouped GEMM
// h.Wl2 with the gate weight fused into the epilogue, and the K-way combine.
#include <algorithm>
#include <type_traits>

#include "gemm_tile.hpp"

namespace momoe {
namespace {

constexpr int BN = 256;  // GEMM columns per tile
constexpr int FN = 2;    // 2x4 waves, each (32 * FM) rows x 64 columns
using WeightOp = TDma;   // expert weights [k][col], k-strided

struct Lin1Args {
  const bf16* x;
  const bf16* w1;
  const int32_t* idx;
  const int32_t* table;
  bf16* h;
  bf16* ab;
  int64_t ab_lo, ab_hi;
  int D, H;
  // backward only (rows >= ab_lo): dL/dh without the gate weight, the gate weights, outputs
  const bf16* u;
  const float* s;
  int64_t ssn, ssm;
  bf16* gz;
  bf16* hst;    // hs in groups of 32 padded sorted rows, [group][ldt features][32]
  int64_t ldt;
  float* gs_part;
  int64_t msum;
  unsigned long long* clk;
};

// Tile = up to 320 (256) rows x (128 `a` columns + the matching 128 `b` columns); a wave owns 32 `a`
// columns and their 32 `b` columns, so the SwiGLU product pairs registers of the same lane.
// BWD = false: forward / recomputation, writes h and/or a|b.  BWD = true: the a|b of the tile
// stay in registers and go straight into the SwiGLU backward.
// G: the row-tile geometry.  The forward takes either; the backward's epilogue needs the registers
// of the fifth fragment row, so it only exists for 256-row tiles and runs on a tile table of its own.
template <bool BWD, class G>
struct Lin1Prog {
  static_assert(!BWD || std::is_same_v<G, StdTiles>, "the SwiGLU backward epilogue fits 256-row tiles only");
  static constexpr int FM = G::FM, BM = G::MAX_ROWS;
  using RowsOp = RDma<G::AROWS>;  // token rows, k-contiguous
  using Ring = StageRing<RowsOp, WeightOp, G::STAGES>;
  static constexpr size_t kLds = Ring::BYTES;
  static constexpr int BNH = BN / 2;
  static_assert(BNH == MOMOE_GS_BLOCK, "gs_part blocks follow the hidden-column tile");
  static_assert(4 * BM * sizeof(float) <= kEpilogueLds, "the dL/ds row sums reuse the staging area");
  struct Prep {
    int32_t tok[RowsOp::NCH];  // tokens of the rows this lane fetches
    int32_t etok[BWD ? FM : 1];  // backward: tokens of the rows this lane holds in the accumulators
    float sv[BWD ? FM : 1];      // and their gate weights
  };
  const Lin1Args& p;
  const int ktiles, wn;

  __device__ __forceinline__ void gather(const TileCoord& t, Prep& g) const {
#pragma unroll
    for (int j = 0; j < RowsOp::NCH; ++j) g.tok[j] = p.idx[t.row0 + min(RowsOp::row_of(j), t.rows - 1)];
    if (BWD) {
#pragma unroll
      for (int i = 0; i < FM; ++i) g.etok[i] = p.idx[t.row0 + min(t.mbase + 32 * i + acc_row(), t.rows - 1)];
    }
  }
  __device__ __forceinline__ void late(const TileCoord& t, Prep& g) const {
    if (BWD) {
#pragma unroll
      for (int i = 0; i < FM; ++i) g.sv[i] = p.s[(int64_t)t.expert * p.ssn + (int64_t)g.etok[i] * p.ssm];
    }
  }
  __device__ __forceinline__ void setup(const TileCoord& t, const Prep& g, RowsOp& A, WeightOp& B) const {
    const int D = p.D, H = p.H;
    const bf16* w = p.w1 + (int64_t)t.expert * D * 2 * H;
    const int j0 = t.tn * BNH;
    A.init(p.x, [&](int, int j) { return (uint32_t)g.tok[j] * (uint32_t)(2 * D); });
    B.init(w, [&](int c) { return (c / BNH) * H + min(j0 + (c % BNH), H - 8); }, 2 * H);
  }
  // epi: store staging; in the backward also the row-sum exchange
  __device__ __forceinline__ void epilogue(const TileCoord& tc, f32x16 (&acc)[FN][FM], const Prep& g, bf16* epi) const {
    if (BWD) epilogue_bwd(tc, acc, g, epi);
    else epilogue_fwd(tc, acc, epi);
  }

  __device__ __forceinline__ void epilogue_fwd(const TileCoord& tc, f32x16 (&acc)[FN][FM], bf16* epi) const {
    const int H = p.H;
    RowStager<1> stager(epi);
    const int j0 = tc.tn * BNH + wn * 32;  // first hidden column of this wave
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if (i >= tc.na) break;  // wave-uniform: no valid row in this fragment row
      float a[4][4], b[4][4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[q][e] = acc[0][i][4 * q + e];
          b[q][e] = acc[1][i][4 * q + e];
        }
      // destination of 8 columns of tile row (tc.mbase + 32 * i)+row in a [*, ld] matrix, or nullptr
      auto dst = [&](bf16* mat, int64_t ld, int col0, bool rows_lo_hi) {
        return [=, *this](int row, int col) -> bf16* {
          const int rl = (tc.mbase + 32 * i) + row;
          const int64_t r = (int64_t)tc.row0 + rl;
          if (rl >= tc.rows || j0 + col >= H) return nullptr;
          if (rows_lo_hi && (r < p.ab_lo || r >= p.ab_hi)) return nullptr;
          return mat + r * ld + col0 + j0 + col;
        };
      };
      if (p.h) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          stager.put(0, q, pack_bf16x4(a[q][0] * b[q][0] * sigmoidf_fast(b[q][0]),
                                       a[q][1] * b[q][1] * sigmoidf_fast(b[q][1]),
                                       a[q][2] * b[q][2] * sigmoidf_fast(b[q][2]),
                                       a[q][3] * b[q][3] * sigmoidf_fast(b[q][3])));
        // h is k-blocked for the next GEMM: this wave's 32 hidden columns are one k-block, so
        // the fragment's rows are consecutive 64-byte pieces of memory
        bf16* hblock = p.h + (int64_t)(j0 >> 5) * p.msum * 32;
        stager.flush([&](int row, int col) -> bf16* {
          const int rl = (tc.mbase + 32 * i) + row;
          if (rl >= tc.rows || j0 >= H) return nullptr;
          return hblock + ((int64_t)tc.row0 + rl) * 32 + col;
        });
      }
      if (p.ab) {
#pragma unroll
        for (int q = 0; q < 4; ++q) stager.put(0, q, pack_bf16x4(a[q][0], a[q][1], a[q][2], a[q][3]));
        stager.flush(dst(p.ab, 2 * H, 0, true));
#pragma unroll
        for (int q = 0; q < 4; ++q) stager.put(0, q, pack_bf16x4(b[q][0], b[q][1], b[q][2], b[q][3]));
        stager.flush(dst(p.ab, 2 * H, H, true));
      }
    }
  }

  // SwiGLU backward on the recomputed a|b (momoe/momoe.py:421-535): with u = dL/dh before the
  // gate weight s,  G_a = s u b sig(b),  G_b = s u a sig(b) (1 + b (1 - sig(b))),
  // hs = s a b sig(b),  and the partial row sum of u a b sig(b) over this tile's columns.
  __device__ __forceinline__ void epilogue_bwd(const TileCoord& tc, f32x16 (&acc)[FN][FM], const Prep& g, bf16* epi) const {
    const int H = p.H;
    RowStager<1> stager(epi);
    float* red = (float*)epi;  // [4 column waves][BM]
    const int j0 = tc.tn * BNH + wn * 32;  // first hidden column of this wave
    auto load_u = [&](int i, bf16x4 (&uq)[4]) {
      const int64_t r = (int64_t)tc.row0 + min((tc.mbase + 32 * i) + acc_row(), tc.rows - 1);
#pragma unroll
      for (int q = 0; q < 4; ++q) uq[q] = *(const bf16x4*)(p.u + r * H + min(j0 + acc_col(q), H - 4));
    };
    RowStager<1> stager1(epi, 1);
    // Rows below the save boundary are not this kernel's: the boundary is moved down to a
    // multiple of 32 rows from the expert's first row (tiles start at such multiples), so that
    // a whole 32-row fragment row is either produced here or by momoe_swiglu_bwd_saved.
    const int rl_lo = p.ab_lo > tc.row0 ? (int)((p.ab_lo - tc.row0) & ~(int64_t)31) : 0;
    float gsums[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      gsums[i] = 0.0f;
      if (i >= tc.na) continue;  // wave-uniform
      bf16x4 uq[4];
      load_u(i, uq);
      const float sv = g.sv[i];
      float gsum = 0.0f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float va[4], vb[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float a = acc[0][i][4 * q + e], b = acc[1][i][4 * q + e];
          const float u = (float)uq[q][e];
          const float sg = sigmoidf_fast(b);
          const float t = b * sg;  // silu(b)
          const float hval = a * t;
          gsum += u * hval;
          const float gh = sv * u;
          va[e] = gh * t;
          // d silu / d b = sg (1 + b (1 - sg)) = sg + t - t sg
          vb[e] = (gh * a) * __builtin_fmaf(-t, sg, sg + t);
          acc[0][i][4 * q + e] = sv * hval;  // a is not needed any more: keep hs in its place
        }
        stager.put(0, q, pack_bf16x4(va[0], va[1], va[2], va[3]));
        stager1.put(0, q, pack_bf16x4(vb[0], vb[1], vb[2], vb[3]));
      }
      const int rl0 = tc.mbase + 32 * i;  // first tile row of this fragment row
      const bool mine = rl0 >= rl_lo;      // wave-uniform
      // gz is k-blocked ([2H/32][Msum][32], the layout dL/dx contracts over): this wave's 32
      // columns of G_a are block j0/32, those of G_b block (H + j0)/32, and a fragment's rows are
      // consecutive 64-byte pieces of memory
      auto dst = [&](int block) {
        bf16* base = p.gz + (int64_t)block * p.msum * 32;
        return [=, *this](int row, int col) -> bf16* {
          const int rl = rl0 + row;
          if (rl >= tc.rows || j0 >= H || !mine) return nullptr;
          return base + ((int64_t)tc.row0 + rl) * 32 + col;
        };
      };
      stager.flush(dst(j0 >> 5));
      stager1.flush(dst((H + j0) >> 5));
      // hs^T: the 32 x 32 fragment goes through the staging area transposed ([column][row],
      // the four 8-row groups of a column permuted so that the two half-waves, which write
      // columns 4 apart, use different banks) and leaves it as 8 consecutive rows of one column
      // per lane.  Rows past the expert's last one are written as zeros: they are the padding
      // the weight-gradient GEMM reads.
      {
        bf16* tst = stager.st;
        const int row = acc_row();
        const bool rowok = rl0 + row < tc.rows;
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int col = acc_col(q) + e;
            const int grp = (row >> 3) ^ ((col >> 2) & 3);
            tst[col * 32 + grp * 8 + (row & 7)] = (bf16)(rowok ? acc[0][i][4 * q + e] : 0.0f);
          }
        const int l = threadIdx.x & 63;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
          const int col = pass * 16 + (l >> 2), rg = l & 3;
          const bf16x8 v = *(const bf16x8*)(tst + col * 32 + ((rg ^ ((col >> 2) & 3)) * 8));
          // the fragment's 32 columns x 32 rows are 2 KiB of consecutive memory
          if (mine && j0 + col < H)
            *(bf16x8*)(p.hst + ((int64_t)((tc.prow0 + rl0) >> 5) * p.ldt + j0 + col) * 32 + rg * 8) = v;
        }
      }
      // the wave's 32 hidden columns lie inside H or outside as a whole (H is a multiple of 32)
      gsums[i] = rl0 + acc_row() < tc.rows && j0 < H ? gsum : 0.0f;
    }
    // every wave is done with its staging area before the row sums overwrite it
    wait_lgkm0();
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const float gg = gsums[i] + __shfl_xor(gsums[i], 32);
      // only the fragment rows this wave owns: the others belong to the other wave row
      if (i < tc.na && (threadIdx.x & 63) < 32) red[wn * BM + (tc.mbase + 32 * i) + acc_row()] = gg;
    }
    wait_lgkm0();  // the row sums are in LDS (a full fence would also wait for the stores above)
    __builtin_amdgcn_s_barrier();
    if ((int)threadIdx.x < tc.rows && (int)threadIdx.x >= rl_lo)
      p.gs_part[(int64_t)tc.tn * p.msum + tc.row0 + threadIdx.x] =
          red[threadIdx.x] + red[BM + threadIdx.x] + red[2 * BM + threadIdx.x] +
          red[3 * BM + threadIdx.x];
    wait_lgkm0();
    __builtin_amdgcn_s_barrier();  // `red` is rewritten by the next tile
  }
};

template <bool BWD, class G>
__device__ __forceinline__ void lin1_swiglu_tiles(const Lin1Args& p) {
  using Prog = Lin1Prog<BWD, G>;
  using Ring = typename Prog::Ring;
  constexpr int FM = Prog::FM;
  Ring ring(dyn_lds());
  // without an h output only rows >= ab_lo are wanted: experts entirely below are skipped
  const int first_tile =
      p.h == nullptr && p.ab_lo > 0 ? TileSched::expert_tile_of_row(p.table, p.ab_lo) : 0;
  TileSched sched(p.table, (p.H + Prog::BNH - 1) / Prog::BNH, Prog::BM, first_tile);
  const int wn = wave_id() & 3;
  const int n_org[FN] = {wn * 32, Prog::BNH + wn * 32};
  Prog prog{p, p.D / kBK, wn};
  run_row_tiles<FM, FN>(prog, sched, ring, n_org);
}

// The forward holds both geometries and follows the tile table it is given.
template <bool BWD>
__global__ __launch_bounds__(kThreads, 2) void lin1_swiglu_kernel(Lin1Args p) {
  const ClockTrace trace(p.clk);
  if constexpr (BWD) {
    lin1_swiglu_tiles<true, StdTiles>(p);
  } else {
    if (TileSched::tile_rows_of(p.table) > StdTiles::MAX_ROWS) lin1_swiglu_tiles<false, TallTiles>(p);
    else lin1_swiglu_tiles<false, StdTiles>(p);
  }
  trace.finish();
}
constexpr size_t kLin1FwdLds = std::max(Lin1Prog<false, TallTiles>::kLds, Lin1Prog<false, StdTiles>::kLds);
constexpr size_t kLin1BwdLds = Lin1Prog<true, StdTiles>::kLds;

struct Lin2Args {
  const bf16* h;
  const bf16* w2;
  const float* s;
  int64_t ssn, ssm;
  const int32_t* idx;
  const int32_t* table;
  bf16* ys;
  int D, H;
  int64_t msum;
  unsigned long long* clk;
};

template <class G>
struct Lin2Prog {
  static constexpr int FM = G::FM;
  using HRowsOp = RBlockedDma<G::AROWS>;  // rows of h, k-blocked
  using Ring = StageRing<HRowsOp, WeightOp, G::STAGES>;
  static constexpr size_t kLds = Ring::BYTES;
  struct Prep {
    int32_t tok[FM];  // tokens of the rows this lane holds in the accumulators
    float sv[FM];     // their gate weights
  };
  const Lin2Args& p;
  const int ktiles, wn;

  __device__ __forceinline__ void gather(const TileCoord& t, Prep& g) const {
#pragma unroll
    for (int i = 0; i < FM; ++i) g.tok[i] = p.idx[t.row0 + min(t.mbase + 32 * i + acc_row(), t.rows - 1)];
  }
  __device__ __forceinline__ void late(const TileCoord& t, Prep& g) const {
#pragma unroll
    for (int i = 0; i < FM; ++i) g.sv[i] = p.s[(int64_t)t.expert * p.ssn + (int64_t)g.tok[i] * p.ssm];
  }
  __device__ __forceinline__ void setup(const TileCoord& t, const Prep&, HRowsOp& A, WeightOp& B) const {
    const int D = p.D, H = p.H;
    const bf16* w = p.w2 + (int64_t)t.expert * H * D;
    const int d0 = t.tn * BN;
    A.init(p.h, p.msum, t.row0, t.rows);
    B.init(w, [&](int c) { return min(d0 + c, D - 8); }, D);
  }
  __device__ __forceinline__ void epilogue(const TileCoord& tc, f32x16 (&acc)[FN][FM], const Prep& g, bf16* epi) const {
    const int D = p.D;
    const RowStager<2> stager(epi);
    const int d0 = tc.tn * BN + wn * 64;  // first output column of this wave
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if (i >= tc.na) break;
      const float sv = g.sv[i];
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          stager.put(f, q, pack_bf16x4(acc[f][i][4 * q] * sv, acc[f][i][4 * q + 1] * sv,
                                       acc[f][i][4 * q + 2] * sv, acc[f][i][4 * q + 3] * sv));
      stager.flush([&](int row, int col) -> bf16* {
        const int rl = (tc.mbase + 32 * i) + row;
        if (rl >= tc.rows || d0 + col >= D) return nullptr;
        return p.ys + ((int64_t)tc.row0 + rl) * D + d0 + col;
      });
    }
  }
};

template <class G>
__device__ __forceinline__ void lin2_scale_tiles(const Lin2Args& p) {
  using Prog = Lin2Prog<G>;
  typename Prog::Ring ring(dyn_lds());
  TileSched sched(p.table, (p.D + BN - 1) / BN, G::MAX_ROWS);
  const int wn = wave_id() & 3;
  const int n_org[FN] = {wn * 64, wn * 64 + 32};
  Prog prog{p, p.H / kBK, wn};
  run_row_tiles<Prog::FM, FN>(prog, sched, ring, n_org);
}

__global__ __launch_bounds__(kThreads, 2) void lin2_scale_kernel(Lin2Args p) {
  const ClockTrace trace(p.clk);
  if (TileSched::tile_rows_of(p.table) > StdTiles::MAX_ROWS) lin2_scale_tiles<TallTiles>(p);
  else lin2_scale_tiles<StdTiles>(p);
  trace.finish();
}
constexpr size_t kLin2Lds = std::max(Lin2Prog<TallTiles>::kLds, Lin2Prog<StdTiles>::kLds);

// out[m] = sum_k rows[inv[m,k]]: one workgroup per token, 16-byte loads, fp32 accumulate.
// The row numbers and then the rows are fetched 8 at a time with unconditional loads (a missing
// pair, inv = -1, is pointed at row 0 and left out of the sum): loads under a branch would be
// waited for one by one.
__global__ __launch_bounds__(256) void combine_kernel(const bf16* __restrict__ rows,
                                                      const int32_t* __restrict__ inv,
                                                      bf16* __restrict__ out, int D, int K,
                                                      int64_t msum) {
  const int64_t m = blockIdx.x;
  for (int c = threadIdx.x; c < D / 8; c += blockDim.x) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int k0 = 0; k0 < K; k0 += 8) {
      int32_t r[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) r[j] = inv[m * K + min(k0 + j, K - 1)];
      bf16x8 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool ok = k0 + j < K && (uint32_t)r[j] < (uint64_t)msum;
        v[j] = *(const bf16x8*)(rows + (int64_t)(ok ? r[j] : 0) * D + c * 8);
        r[j] = ok ? 1 : 0;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += r[j] ? (float)v[j][e] : 0.0f;
    }
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)acc[e];
    *(bf16x8*)(out + m * D + c * 8) = o;
  }
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

inline int check_dims(int64_t M, int64_t D, int64_t H, int64_t N, int64_t Msum) {
  if (M <= 0 || D <= 0 || H <= 0 || N <= 0 || Msum <= 0) return MOMOE_ERR_BAD_ARG;
  if (D % kBK != 0 || H % kBK != 0) return MOMOE_ERR_UNSUPPORTED;
  // per-lane source offsets are 32-bit byte offsets from x / from an expert's weights
  if (Msum >= (1ll << 31) || M * D * 2 >= (1ll << 32) || D * H * 4 >= (1ll << 32))
    return MOMOE_ERR_UNSUPPORTED;
  return MOMOE_OK;
}

}  // namespace
}  // namespace momoe

using namespace momoe;

extern "C" int momoe_lin1_swiglu_fwd(const void* x_MD, const void* Wl1_ND2H,
                                     const int32_t* idx_Msum, const int32_t* tile_table,
                                     void* h_blocked, void* ab_rows, int64_t ab_row_lo,
                                     int64_t ab_row_hi, int64_t M, int64_t D, int64_t H,
                                     int64_t N, int64_t Msum, void* stream) {
  if (!x_MD || !Wl1_ND2H || !idx_Msum || !tile_table || (!h_blocked && !ab_rows))
    return MOMOE_ERR_BAD_ARG;
  if (!aligned16(x_MD) || !aligned16(Wl1_ND2H) || ((uintptr_t)h_blocked & 15) ||
      ((uintptr_t)ab_rows & 15))
    return MOMOE_ERR_BAD_ARG;
  const int st = check_dims(M, D, H, N, Msum);
  if (st != MOMOE_OK) return st;
  Lin1Args a{(const bf16*)x_MD, (const bf16*)Wl1_ND2H, idx_Msum, tile_table, (bf16*)h_blocked,
             (bf16*)ab_rows, ab_row_lo, ab_row_hi, (int)D, (int)H,
             nullptr, nullptr, 0, 0, nullptr, nullptr, 0, nullptr, Msum, clock_trace_buffer()};
  static LdsLimit lds;
  if (!allow_lds(lin1_swiglu_kernel<false>, kLin1FwdLds, lds)) return MOMOE_ERR_LAUNCH;
  lin1_swiglu_kernel<false><<<persistent_grid(), kThreads, kLin1FwdLds, (hipStream_t)stream>>>(a);
  return launch_status();
}

extern "C" int momoe_lin1_swiglu_bwd(const void* x_MD, const void* Wl1_ND2H,
                                     const int32_t* idx_Msum, const int32_t* tile_table,
                                     const void* u_MsumH, const float* s_NM, int64_t s_stride_n,
                                     int64_t s_stride_m, int64_t row_lo, void* gz_blocked,
                                     void* hsT_GH32, int64_t ld_hsT, float* gs_part, int64_t M,
                                     int64_t D, int64_t H, int64_t N, int64_t Msum, void* stream) {
  if (!x_MD || !Wl1_ND2H || !idx_Msum || !tile_table || !u_MsumH || !s_NM || !gz_blocked ||
      !hsT_GH32 || !gs_part)
    return MOMOE_ERR_BAD_ARG;
  if (row_lo < 0 || row_lo > Msum) return MOMOE_ERR_BAD_ARG;
  if (!aligned16(x_MD) || !aligned16(Wl1_ND2H) || ((uintptr_t)u_MsumH & 7) ||
      !aligned16(gz_blocked) || !aligned16(hsT_GH32))
    return MOMOE_ERR_BAD_ARG;
  if (ld_hsT < H || ld_hsT % 8 != 0) return MOMOE_ERR_BAD_ARG;
  const int st = check_dims(M, D, H, N, Msum);
  if (st != MOMOE_OK) return st;
  if (row_lo == Msum) return MOMOE_OK;
  Lin1Args a{(const bf16*)x_MD, (const bf16*)Wl1_ND2H, idx_Msum, tile_table, nullptr, nullptr,
             row_lo, Msum, (int)D, (int)H, (const bf16*)u_MsumH, s_NM, s_stride_n, s_stride_m,
             (bf16*)gz_blocked, (bf16*)hsT_GH32, ld_hsT, gs_part, Msum, clock_trace_buffer()};
  static LdsLimit lds;
  if (!allow_lds(lin1_swiglu_kernel<true>, kLin1BwdLds, lds)) return MOMOE_ERR_LAUNCH;
  lin1_swiglu_kernel<true><<<persistent_grid(), kThreads, kLin1BwdLds, (hipStream_t)stream>>>(a);
  return launch_status();
}

extern "C" int momoe_lin2_scale_fwd(const void* h_blocked, const void* Wl2_NHD, const float* s_NM,
                                    int64_t s_stride_n, int64_t s_stride_m,
                                    const int32_t* idx_Msum, const int32_t* tile_table,
                                    void* ys_MsumD, int64_t M, int64_t D, int64_t H, int64_t N,
                                    int64_t Msum, void* stream) {
  if (!h_blocked || !Wl2_NHD || !s_NM || !idx_Msum || !tile_table || !ys_MsumD)
    return MOMOE_ERR_BAD_ARG;
  if (!aligned16(h_blocked) || !aligned16(Wl2_NHD) || ((uintptr_t)ys_MsumD & 7))
    return MOMOE_ERR_BAD_ARG;
  const int st = check_dims(M, D, H, N, Msum);
  if (st != MOMOE_OK) return st;
  Lin2Args a{(const bf16*)h_blocked, (const bf16*)Wl2_NHD, s_NM, s_stride_n, s_stride_m,
             idx_Msum, tile_table, (bf16*)ys_MsumD, (int)D, (int)H, Msum, clock_trace_buffer()};
  static LdsLimit lds;
  if (!allow_lds(lin2_scale_kernel, kLin2Lds, lds)) return MOMOE_ERR_LAUNCH;
  lin2_scale_kernel<<<persistent_grid(), kThreads, kLin2Lds, (hipStream_t)stream>>>(a);
  return launch_status();
}

extern "C" int momoe_combine(const void* rows_MsumD, const int32_t* inv_MK, void* out_MD,
                             int64_t M, int64_t D, int64_t K, int64_t Msum, void* stream) {
  if (!rows_MsumD || !inv_MK || !out_MD) return MOMOE_ERR_BAD_ARG;
  if (M <= 0 || D <= 0 || K <= 0 || Msum <= 0) return MOMOE_ERR_BAD_ARG;
  if (D % 8 != 0 || M >= (1ll << 31) || Msum >= (1ll << 31)) return MOMOE_ERR_UNSUPPORTED;
  if (!aligned16(rows_MsumD) || !aligned16(out_MD)) return MOMOE_ERR_BAD_ARG;
  combine_kernel<<<(unsigned)M, 256, 0, (hipStream_t)stream>>>(
      (const bf16*)rows_MsumD, inv_MK, (bf16*)out_MD, (int)D, (int)K, Msum);
  return launch_status();
}
