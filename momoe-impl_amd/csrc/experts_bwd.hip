// Backward of the experts, data-gradient side: dL/dh fused with the SwiGLU
// backward and the gate-weight gradient, dL/dx in sorted order, and the scatter
// of the gate-weight gradient into [N, M].
#include "gemm_tile.hpp"

namespace momoe {
namespace {

constexpr int BM = MOMOE_TILE_ROWS;
constexpr int BN = 256;
constexpr int FM = 2, FN = 4;
static_assert(BN == MOMOE_GS_BLOCK, "gs_part blocks follow the column tile");
using RowsA = RDma<BM>;  // sorted / gathered token rows, k-contiguous
using RowsB = RDma<BN>;  // weight rows, k-contiguous (the "NT" GEMMs of the data gradients)
constexpr size_t kBwdLds = gemm_lds_bytes<RowsA, RowsB>();

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
__global__ __launch_bounds__(kThreads, 2) void dgrad_h_swiglu_kernel(DhArgs p) {
  using AOp = RowsA;
  using BOp = RowsB;
  bf16* lds = dyn_lds();
  const int D = p.D, H = p.H;
  const int nb = (H + BN - 1) / BN;
  const TileCoord tc = decode_tile(p.table, nb);
  if (!tc.valid) return;
  const int n0 = tc.tn * BN;
  const bf16* w = p.w2 + (int64_t)tc.expert * H * D;

  AOp A;
  BOp B;
  A.init([&](int r) { return p.gy + (int64_t)p.idx[tc.row0 + min(r, tc.rows - 1)] * D; });
  B.init([&](int r) { return w + (int64_t)min(n0 + r, H - 1) * D; });

  const int wave = threadIdx.x >> 6, wm = wave & 1, wn = wave >> 1;
  const int m_org[FM] = {wm * 64, wm * 64 + 32};
  const int n_org[FN] = {wn * 128, wn * 128 + 32, wn * 128 + 64, wn * 128 + 96};
  f32x16 acc[FN][FM];
  zero_acc<FM, FN>(acc);
  gemm_mainloop<AOp, BOp, FM, FN>(A, B, acc, D / kBK, lds, m_org, n_org);

  __syncthreads();           // every wave is done with the LDS stages
  float* red = (float*)lds;  // [2][BM]
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int rloc = m_org[i] + acc_row();
    float gsum = 0.0f;
    if (rloc < tc.rows) {
      const int64_t r = (int64_t)tc.row0 + rloc;
      const float sv = p.s[(int64_t)tc.expert * p.ssn + (int64_t)p.idx[r] * p.ssm];
      const bf16* abp = r < p.msave ? p.ab_save + r * 2 * H : p.gz + r * 2 * H;
      bf16* gzp = p.gz + r * 2 * H;
      bf16* hsp = p.hs + r * H;
#pragma unroll
      for (int f = 0; f < FN; ++f) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + n_org[f] + acc_col(q);
          if (n >= H) continue;
          const bf16x4 a4 = *(const bf16x4*)(abp + n);
          const bf16x4 b4 = *(const bf16x4*)(abp + H + n);
          float ga[4], gb[4], hv[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float a = (float)a4[e], b = (float)b4[e];
            const float u = acc[f][i][4 * q + e];
            const float sg = sigmoidf_fast(b);
            const float hval = a * b * sg;
            gsum += u * hval;
            const float gh = sv * u;
            ga[e] = gh * b * sg;
            gb[e] = gh * a * sg * (1.0f + b * (1.0f - sg));
            hv[e] = sv * hval;
          }
          store_bf16x4(gzp + n, ga[0], ga[1], ga[2], ga[3]);
          store_bf16x4(gzp + H + n, gb[0], gb[1], gb[2], gb[3]);
          store_bf16x4(hsp + n, hv[0], hv[1], hv[2], hv[3]);
        }
      }
    }
    gsum += __shfl_xor(gsum, 32);
    if ((threadIdx.x & 63) < 32) red[wn * BM + rloc] = gsum;
  }
  __syncthreads();
  if (threadIdx.x < BM && (int)threadIdx.x < tc.rows)
    p.gs_part[(int64_t)tc.tn * p.msum + tc.row0 + threadIdx.x] =
        red[threadIdx.x] + red[BM + threadIdx.x];
}

struct DxArgs {
  const bf16* gz;
  const bf16* w1;
  const int32_t* table;
  bf16* gxs;
  int D, H;
};

// gxs = gz . Wl1^T: contraction over the 2H contiguous columns of both operands.
__global__ __launch_bounds__(kThreads, 2) void dgrad_x_kernel(DxArgs p) {
  using AOp = RowsA;
  using BOp = RowsB;
  bf16* lds = dyn_lds();
  const int D = p.D, H2 = 2 * p.H;
  const int nb = (D + BN - 1) / BN;
  const TileCoord tc = decode_tile(p.table, nb);
  if (!tc.valid) return;
  const int d0 = tc.tn * BN;
  const bf16* w = p.w1 + (int64_t)tc.expert * D * H2;

  AOp A;
  BOp B;
  A.init([&](int r) { return p.gz + ((int64_t)tc.row0 + min(r, tc.rows - 1)) * H2; });
  B.init([&](int r) { return w + (int64_t)min(d0 + r, D - 1) * H2; });

  const int wave = threadIdx.x >> 6, wm = wave & 1, wn = wave >> 1;
  const int m_org[FM] = {wm * 64, wm * 64 + 32};
  const int n_org[FN] = {wn * 128, wn * 128 + 32, wn * 128 + 64, wn * 128 + 96};
  f32x16 acc[FN][FM];
  zero_acc<FM, FN>(acc);
  gemm_mainloop<AOp, BOp, FM, FN>(A, B, acc, H2 / kBK, lds, m_org, n_org);

#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int rloc = m_org[i] + acc_row();
    if (rloc >= tc.rows) continue;
    bf16* out = p.gxs + ((int64_t)tc.row0 + rloc) * D;
#pragma unroll
    for (int f = 0; f < FN; ++f) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int d = d0 + n_org[f] + acc_col(q);
        if (d >= D) continue;
        store_bf16x4(out + d, acc[f][i][4 * q], acc[f][i][4 * q + 1], acc[f][i][4 * q + 2],
                     acc[f][i][4 * q + 3]);
      }
    }
  }
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
  if (Msum >= (1ll << 31) || M * D >= (1ll << 40) || D > (1 << 20) || H > (1 << 20))
    return MOMOE_ERR_UNSUPPORTED;
  return MOMOE_OK;
}

inline unsigned grid_for(int64_t Msum, int64_t N, int64_t nb) {
  const int64_t ub = max_row_tiles(Msum, N, BM) * nb;
  return (unsigned)(cdiv64(ub, 8) * 8);
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
  const unsigned grid = grid_for(Msum, N, cdiv64(H, BN));
  static std::once_flag once;
  allow_lds(dgrad_h_swiglu_kernel, kBwdLds, once);
  dgrad_h_swiglu_kernel<<<grid, kThreads, kBwdLds, (hipStream_t)stream>>>(a);
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
  const unsigned grid = grid_for(Msum, N, cdiv64(D, BN));
  static std::once_flag once;
  allow_lds(dgrad_x_kernel, kBwdLds, once);
  dgrad_x_kernel<<<grid, kThreads, kBwdLds, (hipStream_t)stream>>>(a);
  return launch_status();
}
