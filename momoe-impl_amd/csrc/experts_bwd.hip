// Backward of the experts, data-gradient side: dL/dh (before the gate weight), the SwiGLU
// backward for rows whose pre-activations were saved (the others get theirs in the epilogue of
// the recomputing x.Wl1 GEMM), dL/dx in sorted order, and the scatter of the gate-weight
// gradient into [N, M].
#include <algorithm>

#include "gemm_tile.hpp"

namespace momoe {
namespace {

// Both data-gradient GEMMs hold both row-tile geometries and follow the tile table they are given.
constexpr int BN = 256;
constexpr int FN = 2;    // 2x4 waves, each (32 * FM) rows x 64 columns
using RowsB = RDma<BN>;  // weight rows, k-contiguous (the "NT" GEMMs of the data gradients)

struct DhArgs {
  const bf16* gy;
  const bf16* w2;
  const int32_t* idx;
  const int32_t* table;
  bf16* u;
  int D, H;
  unsigned long long* clk;
};

// u = G_y[idx] . Wl2^T is an "NT" GEMM: both operands are k-contiguous (k = D).
template <class G>
struct DhProg {
  static constexpr int FM = G::FM;
  using RowsA = RDma<G::AROWS>;  // gathered token rows, k-contiguous
  using Ring = StageRing<RowsA, RowsB, G::STAGES>;  // its idle buffer is the store staging
  struct Prep {
    int32_t tok[RowsA::NCH];  // tokens of the rows this lane fetches
  };
  const DhArgs& p;
  const int ktiles, wn;

  __device__ __forceinline__ void gather(const TileCoord& t, Prep& g) const {
#pragma unroll
    for (int j = 0; j < RowsA::NCH; ++j) g.tok[j] = p.idx[t.row0 + min(RowsA::row_of(j), t.rows - 1)];
  }
  __device__ __forceinline__ void late(const TileCoord&, Prep&) const {}
  __device__ __forceinline__ void setup(const TileCoord& t, const Prep& g, RowsA& A, RowsB& B) const {
    const int D = p.D, H = p.H;
    const bf16* w = p.w2 + (int64_t)t.expert * H * D;
    const int n0 = t.tn * BN;
    A.init(p.gy, [&](int, int j) { return (uint32_t)g.tok[j] * (uint32_t)(2 * D); });
    B.init(w, [&](int r, int) { return (uint32_t)min(n0 + r, H - 1) * (uint32_t)(2 * D); });
  }
  __device__ __forceinline__ void epilogue(const TileCoord& tc, f32x16 (&acc)[FN][FM], const Prep&, bf16* epi) const {
    const int H = p.H;
    const RowStager<2> stager(epi);
    const int n0 = tc.tn * BN + wn * 64;  // first hidden column of this wave
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if (i >= tc.na) break;
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          stager.put(f, q, pack_bf16x4(acc[f][i][4 * q], acc[f][i][4 * q + 1],
                                       acc[f][i][4 * q + 2], acc[f][i][4 * q + 3]));
      stager.flush([&](int row, int col) -> bf16* {
        const int rl = (tc.mbase + 32 * i) + row;
        if (rl >= tc.rows || n0 + col >= H) return nullptr;
        return p.u + ((int64_t)tc.row0 + rl) * H + n0 + col;
      });
    }
  }
};

template <class G>
__device__ __forceinline__ void dgrad_h_tiles(const DhArgs& p) {
  using Prog = DhProg<G>;
  typename Prog::Ring ring(dyn_lds());
  TileSched sched(p.table, (p.H + BN - 1) / BN, G::MAX_ROWS);
  const int wn = wave_id() & 3;
  const int n_org[FN] = {wn * 64, wn * 64 + 32};
  Prog prog{p, p.D / kBK, wn};
  run_row_tiles<Prog::FM, FN>(prog, sched, ring, n_org);
}

__global__ __launch_bounds__(kThreads, 2) void dgrad_h_kernel(DhArgs p) {
  const ClockTrace trace(p.clk);
  if (TileSched::tile_rows_of(p.table) > StdTiles::MAX_ROWS) dgrad_h_tiles<TallTiles>(p);
  else dgrad_h_tiles<StdTiles>(p);
  trace.finish();
}
constexpr size_t kDhLds = std::max(DhProg<TallTiles>::Ring::BYTES, DhProg<StdTiles>::Ring::BYTES);

// SwiGLU backward for the sorted rows whose a|b were saved by the forward.  One workgroup per
// group of 32 padded sorted rows (an expert's rows start at a multiple of 32 in padded
// positions, so a group never straddles two experts); it walks the hidden columns 64 at a time:
// thread t holds row t/8 and 8 of the 64 columns, writes its piece of gz row-major, and passes
// its piece of hs through LDS transposed, from where 8 consecutive rows of one column leave per
// thread for the transposed copy of hs.  Rows of the group past the expert's last one become the zero padding.
// A group belongs to this kernel when all of its rows lie below `Msave`; the remaining groups
// (those of the expert that Msave cuts, from the group holding Msave on, and all later experts)
// are produced by momoe_lin1_swiglu_bwd, which applies the same rule.
struct SavedArgs {
  const bf16* ab;
  const bf16* u;
  const float* s;
  int64_t ssn, ssm;
  const int32_t* idx;
  const int32_t* cumsums;
  bf16* gz;
  bf16* hst;
  int64_t ldt;
  float* gs_part;
  int nparts;
  int64_t msum, msave;
  int H, N, M;
};

constexpr int kSavedCols = 64;    // hidden columns per pass
constexpr int kSavedSpan = 256;   // hidden columns per workgroup: blockIdx.y selects the span
static_assert(kSavedSpan % MOMOE_GS_BLOCK == 0 && kSavedSpan % kSavedCols == 0, "spans cover whole parts");

__global__ __launch_bounds__(256) void swiglu_bwd_saved_kernel(SavedArgs p) {
  __shared__ __attribute__((aligned(16))) bf16 tr[2][kSavedCols * 32];  // [pass parity][column][row]
  const int H = p.H, N = p.N;
  const int pg = blockIdx.x * 32;  // first padded position of the group
  // expert whose padded range holds pg: the last e with padded_start(cumsums[e], e) <= pg
  int lo = 0, hi = N;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (padded_start(min(p.cumsums[mid], (int)p.msum), mid) <= pg) lo = mid; else hi = mid;
  }
  const int c0 = min(p.cumsums[lo], (int)p.msum), c1 = min(p.cumsums[lo + 1], (int)p.msum);
  const int local = pg - padded_start(c0, lo);  // rows of the expert before this group
  const int valid = min(32, c1 - c0 - local);   // rows of the group that exist
  if (local < 0 || valid <= 0) return;           // padding between two experts
  const int64_t r0 = (int64_t)c0 + local;        // first sorted row of the group
  if (r0 + valid > p.msave) return;              // not (entirely) below the save boundary

  const int t = threadIdx.x, row = t >> 3, cc = (t & 7) * 8;
  const bool rowok = row < valid;
  const int64_t r = r0 + min(row, valid - 1);
  const int tok = min(max(p.idx[r], 0), p.M - 1);
  const float sv = p.s[(int64_t)lo * p.ssn + (int64_t)tok * p.ssm];
  const bf16* a_row = p.ab + r * 2 * H;
  const bf16* u_row = p.u + r * H;
  float gsum = 0.0f;
  int par = 0;
  const int hbeg = blockIdx.y * kSavedSpan, hend = min(H, hbeg + kSavedSpan);
  for (int h0 = hbeg; h0 < hend; h0 += kSavedCols, par ^= 1) {
    const int c = h0 + cc;
    bf16x8 hv = {0, 0, 0, 0, 0, 0, 0, 0};
    if (c < H) {
      const bf16x8 a8 = *(const bf16x8*)(a_row + c);
      const bf16x8 b8 = *(const bf16x8*)(a_row + H + c);
      const bf16x8 u8 = *(const bf16x8*)(u_row + c);
      bf16x8 ga, gb;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float a = (float)a8[e], b = (float)b8[e], u = (float)u8[e];
        const float sg = sigmoidf_fast(b);
        const float hval = a * b * sg;
        gsum += u * hval;
        const float gh = sv * u;
        ga[e] = (bf16)(gh * b * sg);
        gb[e] = (bf16)(gh * a * sg * (1.0f + b * (1.0f - sg)));
        hv[e] = (bf16)(rowok ? sv * hval : 0.0f);
      }
      if (rowok) {  // gz is k-blocked: [2H/32][Msum][32]
        *(bf16x8*)(p.gz + ((int64_t)(c >> 5) * p.msum + r) * 32 + (c & 31)) = ga;
        *(bf16x8*)(p.gz + ((int64_t)((H + c) >> 5) * p.msum + r) * 32 + (c & 31)) = gb;
      }
    }
    // transposed staging: column-major, the four 8-row groups of a column rotated by the
    // column so that the 8 threads of a row (columns 8 apart) do not share a bank
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int col = cc + e;
      tr[par][col * 32 + (((row >> 3) ^ (col >> 3)) & 3) * 8 + (row & 7)] = hv[e];
    }
    __syncthreads();  // one barrier per pass: the other buffer is rewritten only after the next one
    const int col = t >> 2, rg = t & 3;
    if (h0 + col < H) {
      const bf16x8 v = *(const bf16x8*)(&tr[par][col * 32 + ((rg ^ (col >> 3)) & 3) * 8]);
      *(bf16x8*)(p.hst + ((int64_t)blockIdx.x * p.ldt + h0 + col) * 32 + rg * 8) = v;
    }
  }
  // dL/ds of the row: the 8 threads of a row are consecutive lanes
#pragma unroll
  for (int o = 4; o > 0; o >>= 1) gsum += __shfl_xor(gsum, o);
  // the sum over this workgroup's span goes to part blockIdx.y; the parts that no span owns
  // (there are ceil(H/128) parts and ceil(H/256) spans) are zeroed by the first span
  if (rowok && (t & 7) == 0) p.gs_part[(int64_t)blockIdx.y * p.msum + r] = gsum;
  if (blockIdx.y == 0 && rowok)
    for (int q = gridDim.y + (t & 7); q < p.nparts; q += 8) p.gs_part[(int64_t)q * p.msum + r] = 0.0f;
}

struct DxArgs {
  const bf16* gz;
  const bf16* w1;
  const int32_t* table;
  bf16* gxs;
  int D, H;
  int64_t msum;
  unsigned long long* clk;
};

// gxs = gz . Wl1^T: contraction over the 2H contiguous columns of both operands.
template <class G>
struct DxProg {
  static constexpr int FM = G::FM;
  using BlockedA = RBlockedDma<G::AROWS>;  // sorted rows of the k-blocked gz
  using Ring = StageRing<BlockedA, RowsB, G::STAGES>;
  struct Prep {};
  const DxArgs& p;
  const int ktiles, wn;

  __device__ __forceinline__ void gather(const TileCoord&, Prep&) const {}
  __device__ __forceinline__ void late(const TileCoord&, Prep&) const {}
  __device__ __forceinline__ void setup(const TileCoord& t, const Prep&, BlockedA& A, RowsB& B) const {
    const int D = p.D, H2 = 2 * p.H;
    const bf16* w = p.w1 + (int64_t)t.expert * D * H2;
    const int d0 = t.tn * BN;
    A.init(p.gz, p.msum, t.row0, t.rows);
    B.init(w, [&](int r, int) { return (uint32_t)min(d0 + r, D - 1) * (uint32_t)(2 * H2); });
  }
  __device__ __forceinline__ void epilogue(const TileCoord& tc, f32x16 (&acc)[FN][FM], const Prep&, bf16* epi) const {
    const int D = p.D;
    const RowStager<2> stager(epi);
    const int d0 = tc.tn * BN + wn * 64;  // first output column of this wave
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if (i >= tc.na) break;
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          stager.put(f, q, pack_bf16x4(acc[f][i][4 * q], acc[f][i][4 * q + 1],
                                       acc[f][i][4 * q + 2], acc[f][i][4 * q + 3]));
      stager.flush([&](int row, int col) -> bf16* {
        const int rl = (tc.mbase + 32 * i) + row;
        if (rl >= tc.rows || d0 + col >= D) return nullptr;
        return p.gxs + ((int64_t)tc.row0 + rl) * D + d0 + col;
      });
    }
  }
};

template <class G>
__device__ __forceinline__ void dgrad_x_tiles(const DxArgs& p) {
  using Prog = DxProg<G>;
  typename Prog::Ring ring(dyn_lds());
  TileSched sched(p.table, (p.D + BN - 1) / BN, G::MAX_ROWS);
  const int wn = wave_id() & 3;
  const int n_org[FN] = {wn * 64, wn * 64 + 32};
  Prog prog{p, (2 * p.H) / kBK, wn};
  run_row_tiles<Prog::FM, FN>(prog, sched, ring, n_org);
}

__global__ __launch_bounds__(kThreads, 2) void dgrad_x_kernel(DxArgs p) {
  const ClockTrace trace(p.clk);
  if (TileSched::tile_rows_of(p.table) > StdTiles::MAX_ROWS) dgrad_x_tiles<TallTiles>(p);
  else dgrad_x_tiles<StdTiles>(p);
  trace.finish();
}
constexpr size_t kDxLds = std::max(DxProg<TallTiles>::Ring::BYTES, DxProg<StdTiles>::Ring::BYTES);

__global__ __launch_bounds__(256) void gs_scatter_kernel(const float* __restrict__ part, int nparts,
                                                         const int32_t* __restrict__ idx,
                                                         const int32_t* __restrict__ cumsums,
                                                         float* __restrict__ gs, int M, int N,
                                                         int64_t msum) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  // more pairs than rows: the routing was refused (empty tile table), dL/ds stays zero
  if (r >= msum || r >= cumsums[N] || cumsums[N] > msum) return;
  // expert of row r: the i with cumsums[i] <= r < cumsums[i+1]
  int lo = 0, hi = N;  // invariant: cumsums[lo] <= r < cumsums[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cumsums[mid] <= r) lo = mid; else hi = mid;
  }
  float v = 0.0f;
  for (int q = 0; q < nparts; ++q) v += part[(int64_t)q * msum + r];
  gs[(int64_t)lo * M + idx[r]] = v;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

inline int check_dims(int64_t M, int64_t D, int64_t H, int64_t N, int64_t Msum) {
  if (M <= 0 || D <= 0 || H <= 0 || N <= 0 || Msum <= 0) return MOMOE_ERR_BAD_ARG;
  if (D % kBK != 0 || H % kBK != 0) return MOMOE_ERR_UNSUPPORTED;
  // per-lane source offsets are 32-bit byte offsets from G_y / from an expert's weights
  if (Msum >= (1ll << 31) || M * D * 2 >= (1ll << 32) || D * H * 4 >= (1ll << 32))
    return MOMOE_ERR_UNSUPPORTED;
  return MOMOE_OK;
}

}  // namespace
}  // namespace momoe

using namespace momoe;

extern "C" int momoe_dgrad_h(const void* Gy_MD, const void* Wl2_NHD, const int32_t* idx_Msum,
                             const int32_t* tile_table, void* u_MsumH, int64_t M, int64_t D,
                             int64_t H, int64_t N, int64_t Msum, void* stream) {
  if (!Gy_MD || !Wl2_NHD || !idx_Msum || !tile_table || !u_MsumH) return MOMOE_ERR_BAD_ARG;
  if (!aligned16(Gy_MD) || !aligned16(Wl2_NHD) || !aligned16(u_MsumH)) return MOMOE_ERR_BAD_ARG;
  const int st = check_dims(M, D, H, N, Msum);
  if (st != MOMOE_OK) return st;
  DhArgs a{(const bf16*)Gy_MD, (const bf16*)Wl2_NHD, idx_Msum, tile_table, (bf16*)u_MsumH, (int)D,
           (int)H, clock_trace_buffer()};
  static LdsLimit lds;
  if (!allow_lds(dgrad_h_kernel, kDhLds, lds)) return MOMOE_ERR_LAUNCH;
  dgrad_h_kernel<<<persistent_grid(), kThreads, kDhLds, (hipStream_t)stream>>>(a);
  return launch_status();
}

extern "C" int momoe_swiglu_bwd_saved(const void* ab_save, const void* u_MsumH, const float* s_NM,
                                      int64_t s_stride_n, int64_t s_stride_m,
                                      const int32_t* idx_Msum, const int32_t* cumsums_N1,
                                      int64_t Msave, void* gz_blocked, void* hsT_GH32,
                                      int64_t ld_hsT, float* gs_part, int64_t nparts, int64_t M,
                                      int64_t H, int64_t N, int64_t Msum, void* stream) {
  if (!ab_save || !u_MsumH || !s_NM || !idx_Msum || !cumsums_N1 || !gz_blocked || !hsT_GH32 ||
      !gs_part)
    return MOMOE_ERR_BAD_ARG;
  if (Msave < 0 || Msave > Msum || nparts <= 0 || M <= 0 || H <= 0 || N <= 0 || Msum <= 0)
    return MOMOE_ERR_BAD_ARG;
  if (!aligned16(ab_save) || !aligned16(u_MsumH) || !aligned16(gz_blocked) || !aligned16(hsT_GH32))
    return MOMOE_ERR_BAD_ARG;
  const int64_t mpad = momoe_padded_rows(Msum, N);
  if (ld_hsT < H || ld_hsT % 8 != 0) return MOMOE_ERR_BAD_ARG;
  if (H % 8 != 0 || mpad >= (1ll << 31) || M >= (1ll << 31) || nparts > (1 << 20))
    return MOMOE_ERR_UNSUPPORTED;
  if (Msave == 0) return MOMOE_OK;
  SavedArgs a{(const bf16*)ab_save, (const bf16*)u_MsumH, s_NM, s_stride_n, s_stride_m, idx_Msum,
              cumsums_N1, (bf16*)gz_blocked, (bf16*)hsT_GH32, ld_hsT, gs_part, (int)nparts, Msum,
              Msave, (int)H, (int)N, (int)M};
  const int64_t spans = cdiv64(H, kSavedSpan);
  if (spans > nparts || spans > 65535) return MOMOE_ERR_BAD_ARG;  // nparts = ceil(H / MOMOE_GS_BLOCK)
  swiglu_bwd_saved_kernel<<<dim3((unsigned)(mpad / 32), (unsigned)spans), 256, 0, (hipStream_t)stream>>>(a);
  return launch_status();
}

extern "C" int momoe_gs_scatter(const float* gs_part, int64_t nparts, const int32_t* idx_Msum,
                                const int32_t* cumsums_N1, float* Gs_NM, int64_t M, int64_t N,
                                int64_t Msum, void* stream) {
  if (!gs_part || !idx_Msum || !cumsums_N1 || !Gs_NM) return MOMOE_ERR_BAD_ARG;
  if (nparts <= 0 || M <= 0 || N <= 0 || Msum <= 0) return MOMOE_ERR_BAD_ARG;
  if (Msum >= (1ll << 31) || M >= (1ll << 31)) return MOMOE_ERR_UNSUPPORTED;
  gs_scatter_kernel<<<(unsigned)cdiv64(Msum, 256), 256, 0, (hipStream_t)stream>>>(
      gs_part, (int)nparts, idx_Msum, cumsums_N1, Gs_NM, (int)M, (int)N, Msum);
  return launch_status();
}

extern "C" int momoe_dgrad_x(const void* gz_blocked, const void* Wl1_ND2H,
                             const int32_t* tile_table, void* gxs_MsumD, int64_t M, int64_t D,
                             int64_t H, int64_t N, int64_t Msum, void* stream) {
  if (!gz_blocked || !Wl1_ND2H || !tile_table || !gxs_MsumD) return MOMOE_ERR_BAD_ARG;
  if (!aligned16(gz_blocked) || !aligned16(Wl1_ND2H) || ((uintptr_t)gxs_MsumD & 7))
    return MOMOE_ERR_BAD_ARG;
  const int st = check_dims(M, D, H, N, Msum);
  if (st != MOMOE_OK) return st;
  DxArgs a{(const bf16*)gz_blocked, (const bf16*)Wl1_ND2H, tile_table, (bf16*)gxs_MsumD, (int)D,
           (int)H, Msum, clock_trace_buffer()};
  static LdsLimit lds;
  if (!allow_lds(dgrad_x_kernel, kDxLds, lds)) return MOMOE_ERR_LAUNCH;
  dgrad_x_kernel<<<persistent_grid(), kThreads, kDxLds, (hipStream_t)stream>>>(a);
  return launch_status();
}
