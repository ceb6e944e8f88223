// Backward of the experts, data-gradient side: dL/dh (before the gate weight), the SwiGLU
// backward for rows whose pre-activations were saved (the others get theirs in the epilogue of
// the recomputing x.Wl1 GEMM), dL/dx in sorted order, and the scatter of the gate-weight
// gradient into [N, M].
#include "gemm_tile.hpp"

namespace momoe {
namespace {

constexpr int BM = MOMOE_TILE_ROWS;
constexpr int BN = 256;
constexpr int FM = 4, FN = 2;  // 2x4 waves, each 128 rows x 64 columns
using RowsA = RDma<BM>;  // sorted / gathered token rows, k-contiguous
using RowsB = RDma<BN>;  // weight rows, k-contiguous (the "NT" GEMMs of the data gradients)
using Ring = StageRing<RowsA, RowsB>;
constexpr size_t kBwdLds = Ring::BYTES + kEpilogueLds;  // stage ring + per-wave store staging

struct DhArgs {
  const bf16* gy;
  const bf16* w2;
  const int32_t* idx;
  const int32_t* table;
  bf16* u;
  int D, H;
};

// u = G_y[idx] . Wl2^T is an "NT" GEMM: both operands are k-contiguous (k = D).
struct DhProg {
  struct Prep {
    int32_t tok[RowsA::NCH];  // tokens of the rows this lane fetches
  };
  const DhArgs& p;
  const int ktiles, wn;
  RowStager<2> stager;

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
  __device__ __forceinline__ void epilogue(const TileCoord& tc, f32x16 (&acc)[FN][FM], const Prep&) const {
    const int H = p.H;
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

__global__ __launch_bounds__(kThreads, 2) void dgrad_h_kernel(DhArgs p) {
  Ring ring(dyn_lds());
  TileSched sched(p.table, (p.H + BN - 1) / BN);
  const int wn = (threadIdx.x >> 6) & 3;
  const int n_org[FN] = {wn * 64, wn * 64 + 32};
  DhProg prog{p, p.D / kBK, wn, RowStager<2>(dyn_lds() + kStages * Ring::STAGE)};
  run_row_tiles<FM, FN>(prog, sched, ring, n_org);
}

// SwiGLU backward for the sorted rows whose a|b were saved by the forward: one workgroup per
// row, 8 hidden columns per thread and pass.
struct SavedArgs {
  const bf16* ab;
  const bf16* u;
  const float* s;
  int64_t ssn, ssm;
  const int32_t* idx;
  const int32_t* cumsums;
  bf16* gz;
  bf16* hs;
  float* gs_part;
  int nparts;
  int64_t msum;
  int H, N, M;
};

__global__ __launch_bounds__(256) void swiglu_bwd_saved_kernel(SavedArgs p) {
  const int64_t r = blockIdx.x;
  const int H = p.H;
  __shared__ float s_red[4];
  if (r >= p.cumsums[p.N]) {
    // The routing holds fewer pairs than M*K (a token with fewer than K experts): this sorted
    // row does not exist and its token id was never written.  Its outputs are defined zeros.
    const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int c = threadIdx.x * 8; c < H; c += 256 * 8) {
      *(bf16x8*)(p.gz + r * 2 * H + c) = z;
      *(bf16x8*)(p.gz + r * 2 * H + H + c) = z;
      *(bf16x8*)(p.hs + r * H + c) = z;
    }
    for (int q = threadIdx.x; q < p.nparts; q += 256) p.gs_part[(int64_t)q * p.msum + r] = 0.0f;
    return;
  }
  // expert of row r: the i with cumsums[i] <= r < cumsums[i+1]
  int lo = 0, hi = p.N;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (p.cumsums[mid] <= r) lo = mid; else hi = mid;
  }
  const int tok = min(max(p.idx[r], 0), p.M - 1);
  const float sv = p.s[(int64_t)lo * p.ssn + (int64_t)tok * p.ssm];
  const bf16* a_row = p.ab + r * 2 * H;
  const bf16* u_row = p.u + r * H;
  float gsum = 0.0f;
  for (int c = threadIdx.x * 8; c < H; c += 256 * 8) {
    const bf16x8 a8 = *(const bf16x8*)(a_row + c);
    const bf16x8 b8 = *(const bf16x8*)(a_row + H + c);
    const bf16x8 u8 = *(const bf16x8*)(u_row + c);
    bf16x8 ga, gb, hv;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float a = (float)a8[e], b = (float)b8[e], u = (float)u8[e];
      const float sg = sigmoidf_fast(b);
      const float hval = a * b * sg;
      gsum += u * hval;
      const float gh = sv * u;
      ga[e] = (bf16)(gh * b * sg);
      gb[e] = (bf16)(gh * a * sg * (1.0f + b * (1.0f - sg)));
      hv[e] = (bf16)(sv * hval);
    }
    *(bf16x8*)(p.gz + r * 2 * H + c) = ga;
    *(bf16x8*)(p.gz + r * 2 * H + H + c) = gb;
    *(bf16x8*)(p.hs + r * H + c) = hv;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) gsum += __shfl_xor(gsum, o);
  if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = gsum;
  __syncthreads();
  if (threadIdx.x == 0) p.gs_part[r] = s_red[0] + s_red[1] + s_red[2] + s_red[3];
  // the whole row sum sits in part 0
  for (int q = 1 + threadIdx.x; q < p.nparts; q += 256) p.gs_part[(int64_t)q * p.msum + r] = 0.0f;
}

struct DxArgs {
  const bf16* gz;
  const bf16* w1;
  const int32_t* table;
  bf16* gxs;
  int D, H;
};

// gxs = gz . Wl1^T: contraction over the 2H contiguous columns of both operands.
struct DxProg {
  struct Prep {};
  const DxArgs& p;
  const int ktiles, wn;
  RowStager<2> stager;

  __device__ __forceinline__ void gather(const TileCoord&, Prep&) const {}
  __device__ __forceinline__ void late(const TileCoord&, Prep&) const {}
  __device__ __forceinline__ void setup(const TileCoord& t, const Prep&, RowsA& A, RowsB& B) const {
    const int D = p.D, H2 = 2 * p.H;
    const bf16* w = p.w1 + (int64_t)t.expert * D * H2;
    const int d0 = t.tn * BN;
    A.init(p.gz + (int64_t)t.row0 * H2, [&](int r, int) { return (uint32_t)(min(r, t.rows - 1) * 2 * H2); });
    B.init(w, [&](int r, int) { return (uint32_t)min(d0 + r, D - 1) * (uint32_t)(2 * H2); });
  }
  __device__ __forceinline__ void epilogue(const TileCoord& tc, f32x16 (&acc)[FN][FM], const Prep&) const {
    const int D = p.D;
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

__global__ __launch_bounds__(kThreads, 2) void dgrad_x_kernel(DxArgs p) {
  Ring ring(dyn_lds());
  TileSched sched(p.table, (p.D + BN - 1) / BN);
  const int wn = (threadIdx.x >> 6) & 3;
  const int n_org[FN] = {wn * 64, wn * 64 + 32};
  DxProg prog{p, (2 * p.H) / kBK, wn, RowStager<2>(dyn_lds() + kStages * Ring::STAGE)};
  run_row_tiles<FM, FN>(prog, sched, ring, n_org);
}

__global__ __launch_bounds__(256) void gs_scatter_kernel(const float* __restrict__ part, int nparts,
                                                         const int32_t* __restrict__ idx,
                                                         const int32_t* __restrict__ cumsums,
                                                         float* __restrict__ gs, int M, int N,
                                                         int64_t msum) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= msum || r >= cumsums[N]) return;
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
           (int)H};
  static std::once_flag once;
  allow_lds(dgrad_h_kernel, kBwdLds, once);
  dgrad_h_kernel<<<persistent_grid(), kThreads, kBwdLds, (hipStream_t)stream>>>(a);
  return launch_status();
}

extern "C" int momoe_swiglu_bwd_saved(const void* ab_save, const void* u_MsumH, const float* s_NM,
                                      int64_t s_stride_n, int64_t s_stride_m,
                                      const int32_t* idx_Msum, const int32_t* cumsums_N1,
                                      int64_t Msave, void* gz_Msum2H, void* hs_MsumH,
                                      float* gs_part, int64_t nparts, int64_t M, int64_t H,
                                      int64_t N, int64_t Msum, void* stream) {
  if (!ab_save || !u_MsumH || !s_NM || !idx_Msum || !cumsums_N1 || !gz_Msum2H || !hs_MsumH ||
      !gs_part)
    return MOMOE_ERR_BAD_ARG;
  if (Msave < 0 || Msave > Msum || nparts <= 0 || M <= 0 || H <= 0 || N <= 0 || Msum <= 0)
    return MOMOE_ERR_BAD_ARG;
  if (!aligned16(ab_save) || !aligned16(u_MsumH) || !aligned16(gz_Msum2H) || !aligned16(hs_MsumH))
    return MOMOE_ERR_BAD_ARG;
  if (H % 8 != 0 || Msum >= (1ll << 31) || M >= (1ll << 31) || nparts > (1 << 20))
    return MOMOE_ERR_UNSUPPORTED;
  if (Msave == 0) return MOMOE_OK;
  SavedArgs a{(const bf16*)ab_save, (const bf16*)u_MsumH, s_NM, s_stride_n, s_stride_m, idx_Msum,
              cumsums_N1, (bf16*)gz_Msum2H, (bf16*)hs_MsumH, gs_part, (int)nparts, Msum, (int)H,
              (int)N, (int)M};
  swiglu_bwd_saved_kernel<<<(unsigned)Msave, 256, 0, (hipStream_t)stream>>>(a);
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

extern "C" int momoe_dgrad_x(const void* gz_Msum2H, const void* Wl1_ND2H,
                             const int32_t* tile_table, void* gxs_MsumD, int64_t M, int64_t D,
                             int64_t H, int64_t N, int64_t Msum, void* stream) {
  if (!gz_Msum2H || !Wl1_ND2H || !tile_table || !gxs_MsumD) return MOMOE_ERR_BAD_ARG;
  if (!aligned16(gz_Msum2H) || !aligned16(Wl1_ND2H) || ((uintptr_t)gxs_MsumD & 7))
    return MOMOE_ERR_BAD_ARG;
  const int st = check_dims(M, D, H, N, Msum);
  if (st != MOMOE_OK) return st;
  DxArgs a{(const bf16*)gz_Msum2H, (const bf16*)Wl1_ND2H, tile_table, (bf16*)gxs_MsumD, (int)D,
           (int)H};
  static std::once_flag once;
  allow_lds(dgrad_x_kernel, kBwdLds, once);
  dgrad_x_kernel<<<persistent_grid(), kThreads, kBwdLds, (hipStream_t)stream>>>(a);
  return launch_status();
}
