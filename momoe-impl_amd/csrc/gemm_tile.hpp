// Workgroup-level bf16 GEMM building blocks for gfx950 (CDNA4).
//
// A workgroup of 4 wavefronts computes a BM x BN fp32 tile with
// v_mfma_f32_32x32x16_bf16.  Both MFMA inputs want, per lane, 8 consecutive
// k-values of one row (lane%32 = row, lane/32 = which group of 8 k's).  Two
// kinds of operand tile feed that:
//
//   ROperand  - "k-contiguous": the operand is stored [row][k] in global memory.
//               Staged in LDS as [ROWS][BK+8]; a fragment is one ds_read_b128.
//   TOperand  - "k-strided": the operand is stored [k][col] (the layout of the
//               expert weights in the forward GEMMs, and of everything in the
//               weight-gradient GEMMs).  Staged in LDS as [BK][COLS+16]; a
//               fragment is two ds_read_b64_tr_b16, the gfx950 LDS transpose
//               read: within each group of 16 lanes, lane i supplies the
//               address of 4 consecutive columns of k-row i/4 (columns
//               4*(i%4)..+3) and receives column i of those 4 k-rows.
//
// The MFMA is issued with the N-side fragment as its first input and the M-side
// fragment as its second, so each lane ends up holding, for ONE tile row
// (lane%32), groups of 4 consecutive columns: register r of the 16 holds
// column 8*(r/4) + 4*(lane/32) + r%4.  Row-wise epilogues (per-row scale,
// SwiGLU pairing, row reductions) are then lane-local and stores are 8-byte.
#pragma once
#include "common.hpp"

namespace momoe {

constexpr int kBK = 32;  // k-extent of one LDS stage

__device__ __forceinline__ bf16x4 lds_read_tr4(const bf16* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)p);
}

__device__ __forceinline__ f32x16 mfma32(bf16x8 first, bf16x8 second, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(first, second, c, 0, 0, 0);
}

template <int ROWS>
struct ROperand {
  static_assert(ROWS % 64 == 0, "ROWS must be a multiple of 64");
  static constexpr int LD = kBK + 8;
  static constexpr int CPR = kBK / 8;             // 16-byte chunks per row
  static constexpr int ROWSTEP = kThreads / CPR;  // rows covered by one pass of the workgroup
  static constexpr int NCH = ROWS / ROWSTEP;
  static constexpr int LDS_ELEMS = ROWS * LD;
  const bf16* ptr[NCH];
  u32x4 stage[NCH];

  // rowptr(r) -> global pointer to k=0 of tile row r (must be a readable row for every r < ROWS)
  template <class RowPtr>
  __device__ __forceinline__ void init(RowPtr rowptr) {
    const int kc = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int j = 0; j < NCH; ++j) ptr[j] = rowptr(r + j * ROWSTEP) + kc * 8;
  }
  __device__ __forceinline__ void load(int kt) {
#pragma unroll
    for (int j = 0; j < NCH; ++j) stage[j] = *(const u32x4*)(ptr[j] + kt * kBK);
  }
  __device__ __forceinline__ void store(bf16* lds) const {
    const int kc = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int j = 0; j < NCH; ++j) *(u32x4*)(lds + (r + j * ROWSTEP) * LD + kc * 8) = stage[j];
  }
  // 32 rows starting at r0, k-step kk (16 k-values)
  static __device__ __forceinline__ bf16x8 frag(const bf16* lds, int r0, int kk) {
    const int l = threadIdx.x & 63;
    return *(const bf16x8*)(lds + (r0 + (l & 31)) * LD + kk * 16 + 8 * (l >> 5));
  }
};

template <int COLS>
struct TOperand {
  static_assert(COLS % 64 == 0, "COLS must be a multiple of 64");
  static constexpr int LD = COLS + 16;
  static constexpr int CPR = COLS / 8;
  static constexpr int KSTEP = kThreads / CPR;  // k-rows covered by one pass of the workgroup
  static constexpr int NCH = kBK / KSTEP;
  static_assert(NCH >= 1, "tile too narrow for this stage depth");
  static constexpr int LDS_ELEMS = kBK * LD;
  const bf16* ptr[NCH];
  u32x4 stage[NCH];
  int64_t kstride;
  bool ok;

  // colptr(c) -> global pointer to (k=0, tile column c) for c a multiple of 8, or
  // nullptr when those 8 columns lie outside the matrix (they are then zero-filled).
  // ld = elements between consecutive k-rows in global memory.
  template <class ColPtr>
  __device__ __forceinline__ void init(ColPtr colptr, int64_t ld) {
    const int cc = threadIdx.x % CPR, kr = threadIdx.x / CPR;
    const bf16* base = colptr(cc * 8);
    ok = base != nullptr;
#pragma unroll
    for (int j = 0; j < NCH; ++j) ptr[j] = base + (int64_t)(kr + j * KSTEP) * ld;
    kstride = (int64_t)kBK * ld;
  }
  __device__ __forceinline__ void load(int kt) {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      if (ok) stage[j] = *(const u32x4*)(ptr[j] + kt * kstride);
      else stage[j] = u32x4{0, 0, 0, 0};
    }
  }
  __device__ __forceinline__ void store(bf16* lds) const {
    const int cc = threadIdx.x % CPR, kr = threadIdx.x / CPR;
#pragma unroll
    for (int j = 0; j < NCH; ++j) *(u32x4*)(lds + (kr + j * KSTEP) * LD + cc * 8) = stage[j];
  }
  // 32 columns starting at c0, k-step kk (16 k-values)
  static __device__ __forceinline__ bf16x8 frag(const bf16* lds, int c0, int kk) {
    const int l = threadIdx.x & 63;
    const int krow = kk * 16 + 8 * (l >> 5) + ((l & 15) >> 2);
    const int col = c0 + 16 * ((l & 31) >> 4) + 4 * (l & 3);
    const bf16* p = lds + krow * LD + col;
    const bf16x4 lo = lds_read_tr4(p);
    const bf16x4 hi = lds_read_tr4(p + 4 * LD);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
};

// acc[fn][fm] += Bfrag[fn] x Afrag[fm] over `ktiles` stages of kBK.
// `m_org[fm]` / `n_org[fn]` are the LDS row (or column) origins of this wave's 32-wide
// fragments inside the A / B tile.  LDS is double-buffered: one barrier per stage.
template <class AOp, class BOp, int FM, int FN>
__device__ __forceinline__ void gemm_mainloop(AOp& A, BOp& B, f32x16 (&acc)[FN][FM], int ktiles,
                                              bf16* lds, const int (&m_org)[FM],
                                              const int (&n_org)[FN]) {
  constexpr int STAGE = AOp::LDS_ELEMS + BOp::LDS_ELEMS;
  A.load(0);
  B.load(0);
  A.store(lds);
  B.store(lds + AOp::LDS_ELEMS);
  __syncthreads();
  for (int kt = 0; kt < ktiles; ++kt) {
    const bf16* la = lds + (kt & 1) * STAGE;
    const bf16* lb = la + AOp::LDS_ELEMS;
    const bool more = kt + 1 < ktiles;
    if (more) {
      A.load(kt + 1);
      B.load(kt + 1);
    }
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      bf16x8 af[FM], bf[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) af[i] = AOp::frag(la, m_org[i], kk);
#pragma unroll
      for (int j = 0; j < FN; ++j) bf[j] = BOp::frag(lb, n_org[j], kk);
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int i = 0; i < FM; ++i) acc[j][i] = mfma32(bf[j], af[i], acc[j][i]);
    }
    if (more) {
      bf16* wa = lds + ((kt + 1) & 1) * STAGE;
      A.store(wa);
      B.store(wa + AOp::LDS_ELEMS);
    }
    __syncthreads();
  }
}

template <int FM, int FN>
__device__ __forceinline__ void zero_acc(f32x16 (&acc)[FN][FM]) {
#pragma unroll
  for (int j = 0; j < FN; ++j)
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][i][r] = 0.0f;
}

// Position of accumulator quad q (registers 4q..4q+3) of a 32x32 fragment for this lane:
// tile-local row = lane%32, first of 4 consecutive columns = 8*q + 4*(lane/32).
__device__ __forceinline__ int acc_row() { return threadIdx.x & 31; }
__device__ __forceinline__ int acc_col(int q) { return 8 * q + 4 * ((threadIdx.x & 63) >> 5); }

__device__ __forceinline__ void store_bf16x4(bf16* p, float a, float b, float c, float d) {
  bf16x4 v = {(bf16)a, (bf16)b, (bf16)c, (bf16)d};
  *(bf16x4*)p = v;
}

}  // namespace momoe
