// Backward of the experts, data-gradient side: dL/dh fused with the SwiGLU
// backward and the gate-weight gradient, dL/dx in sorted order, and the scatter
// of the gate-weight gradient into [N, M].
#include "gemm_tile.hpp"

namespace momoe {
namespace {

constexpr int BM = MOMOE_TILE_ROWS;
constexpr int BN = 256;
constexpr int FM = 4, FN = 2;  // 2x4 waves, each 128 rows x 64 columns
static_assert(BN == MOMOE_GS_BLOCK, "gs_part blocks follow the column tile");
using RowsA = RDma<BM>;  // sorted / gathered token rows, k-contiguous
using RowsB = RDma<BN>;  // weight rows, k-contiguous (the "NT" GEMMs of the data gradients)
using Ring = StageRing<RowsA, RowsB>;
constexpr size_t kBwdLds = Ring::BYTES + kEpilogueLds;  // stage ring + per-wave store staging
static_assert(4 * BM * sizeof(float) <= kEpilogueLds, "the dL/ds row sums reuse the staging area");

struct DhArgs {
  const bf16* gy;
  const bf16* w2;
  const float* s;
  int64_t ssn, ssm;
  const int32_t* idx;
  const int32_t* table;
  const bf16* ab_save;
  int64_t msave;
  bf16* gz;
  bf16* hs;
  float* gs_part;
  int64_t msum;
  int D, H;
};

// u = G_y[idx] . Wl2^T is an "NT" GEMM: both operands are k-contiguous (k = D).
struct DhProg {
  struct Prep {
    int32_t tok[RowsA::NCH];  // tokens of the rows this lane fetches
    int32_t etok[FM];         // tokens of the rows this lane holds in the accumulators
    float sv[FM];             // their gate weights
  };
  const DhArgs& p;
  const int ktiles, wn;
  const int (&m_org)[FM];
  bf16* epi;  // store staging, later the row-sum exchange

  __device__ __forceinline__ void gather(const TileCoord& t, Prep& g) const {
#pragma unroll
    for (int j = 0; j < RowsA::NCH; ++j) g.tok[j] = p.idx[t.row0 + min(RowsA::row_of(j), t.rows - 1)];
#pragma unroll
    for (int i = 0; i < FM; ++i) g.etok[i] = p.idx[t.row0 + min(m_org[i] + acc_row(), t.rows - 1)];
  }
  __device__ __forceinline__ void late(const TileCoord& t, Prep& g) const {
#pragma unroll
    for (int i = 0; i < FM; ++i) g.sv[i] = p.s[(int64_t)t.expert * p.ssn + (int64_t)g.etok[i] * p.ssm];
  }
  __device__ __forceinline__ void setup(const TileCoord& t, const Prep& g, RowsA& A, RowsB& B) const {
    const int D = p.D, H = p.H;
    const bf16* w = p.w2 + (int64_t)t.expert * H * D;
    const int n0 = t.tn * BN;
    A.init(p.gy, [&](int, int j) { return (uint32_t)g.tok[j] * (uint32_t)(2 * D); });
    B.init(w, [&](int r, int) { return (uint32_t)min(n0 + r, H - 1) * (uint32_t)(2 * D); });
  }
  __device__ __forceinline__ void epilogue(const TileCoord& tc, f32x16 (&acc)[FN][FM], const Prep& g) const {
    const int H = p.H;
    float* red = (float*)epi;  // [4 column waves][BM], shares the store staging area
    RowStager<1> stage0(epi, 0), stage1(epi, 1);
    const int n0 = tc.tn * BN + wn * 64;  // first hidden column of this wave
    float gsums[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      gsums[i] = 0.0f;
      if (m_org[i] >= tc.rows) continue;  // wave-uniform
      const int rloc = min(m_org[i] + acc_row(), tc.rows - 1);
      const int64_t r = (int64_t)tc.row0 + rloc;
      const float sv = g.sv[i];
      const bf16* abp = r < p.msave ? p.ab_save + r * 2 * H : p.gz + r * 2 * H;
      float gsum = 0.0f;
#pragma unroll
      for (int f = 0; f < FN; ++f) {
        // a|b of the fragment are fetched before anything is stored: the stores go to the
        // buffer the loads come from, so they could not be hoisted above them later
        bf16x4 a4[4], b4[4], hv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = min(n0 + 32 * f + acc_col(q), H - 4);
          a4[q] = *(const bf16x4*)(abp + n);
          b4[q] = *(const bf16x4*)(abp + H + n);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const bool incol = n0 + 32 * f + acc_col(q) < H;
          float va[4], vb[4], vh[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float a = (float)a4[q][e], b = (float)b4[q][e];
            const float u = acc[f][i][4 * q + e];
            const float sg = sigmoidf_fast(b);
            const float hval = a * b * sg;
            gsum += incol ? u * hval : 0.0f;
            const float gh = sv * u;
            va[e] = gh * b * sg;
            vb[e] = gh * a * sg * (1.0f + b * (1.0f - sg));
            vh[e] = sv * hval;
          }
          stage0.put(0, q, pack_bf16x4(va[0], va[1], va[2], va[3]));
          stage1.put(0, q, pack_bf16x4(vb[0], vb[1], vb[2], vb[3]));
          hv[q] = pack_bf16x4(vh[0], vh[1], vh[2], vh[3]);
        }
        auto dst = [&](bf16* mat, int64_t ld, int col0) {
          return [=, *this](int row, int col) -> bf16* {
            const int rl = m_org[i] + row;
            if (rl >= tc.rows || n0 + 32 * f + col >= H) return nullptr;
            return mat + ((int64_t)tc.row0 + rl) * ld + col0 + n0 + 32 * f + col;
          };
        };
        stage0.flush(dst(p.gz, 2 * H, 0));
        stage1.flush(dst(p.gz, 2 * H, H));
#pragma unroll
        for (int q = 0; q < 4; ++q) stage0.put(0, q, hv[q]);
        stage0.flush(dst(p.hs, H, 0));
      }
      gsums[i] = m_org[i] + acc_row() < tc.rows ? gsum : 0.0f;
    }
    // every wave is done with its staging area before the row sums overwrite it
    wait_lgkm0();
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const float gg = gsums[i] + __shfl_xor(gsums[i], 32);
      if ((threadIdx.x & 63) < 32) red[wn * BM + m_org[i] + acc_row()] = gg;
    }
    wait_lgkm0();  // the row sums are in LDS (a full fence would also wait for the stores above)
    __builtin_amdgcn_s_barrier();
    if ((int)threadIdx.x < tc.rows)
      p.gs_part[(int64_t)tc.tn * p.msum + tc.row0 + threadIdx.x] =
          red[threadIdx.x] + red[BM + threadIdx.x] + red[2 * BM + threadIdx.x] +
          red[3 * BM + threadIdx.x];
    wait_lgkm0();
    __builtin_amdgcn_s_barrier();  // `red` is rewritten by the next tile
  }
};

__global__ __launch_bounds__(kThreads, 2) void dgrad_h_swiglu_kernel(DhArgs p) {
  Ring ring(dyn_lds());
  TileSched sched(p.table, (p.H + BN - 1) / BN);
  const int wave = threadIdx.x >> 6, wm = wave >> 2, wn = wave & 3;
  const int m_org[FM] = {wm * 128, wm * 128 + 32, wm * 128 + 64, wm * 128 + 96};
  const int n_org[FN] = {wn * 64, wn * 64 + 32};
  DhProg prog{p, p.D / kBK, wn, m_org, dyn_lds() + kStages * Ring::STAGE};
  run_row_tiles<FM, FN>(prog, sched, ring, m_org, n_org);
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
  const int (&m_org)[FM];
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
      if (m_org[i] >= tc.rows) break;
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          stager.put(f, q, pack_bf16x4(acc[f][i][4 * q], acc[f][i][4 * q + 1],
                                       acc[f][i][4 * q + 2], acc[f][i][4 * q + 3]));
      stager.flush([&](int row, int col) -> bf16* {
        const int rl = m_org[i] + row;
        if (rl >= tc.rows || d0 + col >= D) return nullptr;
        return p.gxs + ((int64_t)tc.row0 + rl) * D + d0 + col;
      });
    }
  }
};

__global__ __launch_bounds__(kThreads, 2) void dgrad_x_kernel(DxArgs p) {
  Ring ring(dyn_lds());
  TileSched sched(p.table, (p.D + BN - 1) / BN);
  const int wave = threadIdx.x >> 6, wm = wave >> 2, wn = wave & 3;
  const int m_org[FM] = {wm * 128, wm * 128 + 32, wm * 128 + 64, wm * 128 + 96};
  const int n_org[FN] = {wn * 64, wn * 64 + 32};
  DxProg prog{p, (2 * p.H) / kBK, wn, m_org, RowStager<2>(dyn_lds() + kStages * Ring::STAGE)};
  run_row_tiles<FM, FN>(prog, sched, ring, m_org, n_org);
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

extern "C" int momoe_dgrad_h_swiglu_bwd(const void* Gy_MD, const void* Wl2_NHD, const float* s_NM,
                                        int64_t s_stride_n, int64_t s_stride_m,
                                        const int32_t* idx_Msum, const int32_t* tile_table,
                                        const void* ab_save, int64_t Msave, void* gz_Msum2H,
                                        void* hs_MsumH, float* gs_part, int64_t M, int64_t D,
                                        int64_t H, int64_t N, int64_t Msum, void* stream) {
  if (!Gy_MD || !Wl2_NHD || !s_NM || !idx_Msum || !tile_table || !gz_Msum2H || !hs_MsumH ||
      !gs_part)
    return MOMOE_ERR_BAD_ARG;
  if (Msave < 0 || Msave > Msum || (Msave > 0 && !ab_save)) return MOMOE_ERR_BAD_ARG;
  if (!aligned16(Gy_MD) || !aligned16(Wl2_NHD) || ((uintptr_t)ab_save & 7) ||
      ((uintptr_t)gz_Msum2H & 7) || ((uintptr_t)hs_MsumH & 7))
    return MOMOE_ERR_BAD_ARG;
  const int st = check_dims(M, D, H, N, Msum);
  if (st != MOMOE_OK) return st;
  DhArgs a{(const bf16*)Gy_MD, (const bf16*)Wl2_NHD, s_NM, s_stride_n, s_stride_m, idx_Msum,
           tile_table, (const bf16*)ab_save, Msave, (bf16*)gz_Msum2H, (bf16*)hs_MsumH, gs_part,
           Msum, (int)D, (int)H};
  static std::once_flag once;
  allow_lds(dgrad_h_swiglu_kernel, kBwdLds, once);
  dgrad_h_swiglu_kernel<<<persistent_grid(), kThreads, kBwdLds, (hipStream_t)stream>>>(a);
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
