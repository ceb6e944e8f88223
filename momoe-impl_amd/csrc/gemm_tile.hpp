// Workgroup-level bf16 GEMM building blocks for gfx950 (CDNA4).
//
// A workgroup of 4 wavefronts computes a BM x BN fp32 tile with
// v_mfma_f32_32x32x16_bf16.  Both MFMA inputs want, per lane, 8 consecutive
// k-values of one row (lane%32 = row, lane/32 = which group of 8 k's).  Two
// kinds of operand tile feed that:
//
//   RDma  - "k-contiguous": the operand is stored [row][k] in global memory.
//           LDS stage [ROWS][32]; a fragment is one ds_read_b128.
//   TDma  - "k-strided": the operand is stored [k][col] (the layout of the
//           expert weights in the forward GEMMs, and of everything in the
//           weight-gradient GEMMs).  LDS stage [32][COLS]; a fragment is two
//           ds_read_b64_tr_b16, the gfx950 LDS transpose read: within each
//           group of 16 lanes, lane i supplies the address of 4 consecutive
//           columns of k-row i/4 (columns 4*(i%4)..+3) and receives column i
//           of those 4 k-rows.
//
// Global memory goes straight to LDS with global_load_lds_dwordx4 (no VGPR
// staging): one wave instruction deposits 64 x 16 bytes contiguously.  Since
// every lane chooses its own global address, the LDS image is swizzled by
// permuting WHICH 16-byte piece each lane fetches: rows keep their natural,
// unpadded pitch, and the fragment reads above are bank-conflict free.  The same
// freedom does all predication: a lane that would read outside the matrix is
// pointed at a clamped row/column (results masked at the store) or, where exact
// zeros are needed along k, at a 16-byte block of zeros.
//
// The k-loop runs a 3-stage ring: while stage t is consumed, the loads of t+1
// and t+2 are in flight; one s_barrier per stage.
//
// The MFMA is issued with the N-side fragment as its first input and the M-side
// fragment as its second, so each lane ends up holding, for ONE tile row
// (lane%32), groups of 4 consecutive columns: register r of the 16 holds
// column 8*(r/4) + 4*(lane/32) + r%4.  Row-wise epilogues (per-row scale,
// SwiGLU pairing, row reductions) are then lane-local and stores are 8-byte.
#pragma once
#include <mutex>

#include "common.hpp"

namespace momoe {

constexpr int kBK = 32;     // k-extent of one LDS stage
constexpr int kStages = 3;  // LDS ring depth
constexpr int kChunkElems = 512;  // one wave-wide 16-byte-per-lane deposit = 1 KiB

static __device__ __attribute__((aligned(16))) const uint32_t kZeroChunk[4] = {0, 0, 0, 0};

__device__ __forceinline__ const bf16* zero_chunk() { return (const bf16*)kZeroChunk; }

// 16 bytes per lane, global -> LDS.  `lds_wave_base` must be wave-uniform; lane L's bytes
// land at lds_wave_base + 16*L.  Completion is tracked by vmcnt.  Issued as inline
// assembly so that the compiler's own wait-count insertion does not know about the
// transfer: with the builtin it forces vmcnt(0) in front of the LDS transpose reads,
// which serialises the ring.  Ordering is therefore entirely manual: wait_vmcnt<>() +
// s_barrier before a stage is read, s_barrier before it is overwritten.
__device__ __forceinline__ void dma16(const bf16* g, bf16* lds_wave_base) {
  const uint32_t lds_addr = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) bf16*)lds_wave_base);
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_addr)
               : "memory");
}

// wait until at most N vector-memory operations of this wave are outstanding
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

__device__ __forceinline__ bf16x4 lds_read_tr4(const bf16* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)p);
}

__device__ __forceinline__ f32x16 mfma32(bf16x8 first, bf16x8 second, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(first, second, c, 0, 0, 0);
}

// ---- k-contiguous operand -------------------------------------------------------------
// LDS stage: row r at elements [32r, 32r+32); its four 16-byte k-pieces are stored at
// position piece ^ ((r>>1)&3), which spreads 8 consecutive rows of one k-piece over all banks.
template <int ROWS>
struct RDma {
  static_assert(ROWS % 64 == 0, "ROWS must be a multiple of 64");
  static constexpr int NCH = ROWS / 64;  // deposits per wave per stage (16 rows each)
  static constexpr int LDS_ELEMS = ROWS * kBK;
  const bf16* ptr[NCH];

  // rowptr(r) -> global pointer to k=0 of tile row r; must be readable for every r < ROWS
  template <class RowPtr>
  __device__ __forceinline__ void init(RowPtr rowptr) {
    const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int row = (j * 4 + w) * 16 + (l >> 2);
      const int piece = (l & 3) ^ ((row >> 1) & 3);
      ptr[j] = rowptr(row) + piece * 8;
    }
  }
  __device__ __forceinline__ void issue(int kt, bf16* stage) {
    const int w = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < NCH; ++j) dma16(ptr[j] + kt * kBK, stage + (j * 4 + w) * kChunkElems);
  }
  // 32 rows starting at r0 (multiple of 32), k-step kk (16 k-values)
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int r0, int kk) {
    const int l = threadIdx.x & 63;
    const int row = r0 + (l & 31);
    const int piece = (2 * kk + (l >> 5)) ^ ((row >> 1) & 3);
    return *(const bf16x8*)(stage + row * kBK + piece * 8);
  }
};

// ---- k-strided operand ----------------------------------------------------------------
// LDS stage: k-row k at elements [COLS*k, COLS*(k+1)); 16-byte piece p of the row is stored
// at position p ^ (2*(k&3)), so the 4 k-rows x 32 bytes that a 16-lane group of the
// transpose read touches fall into 4 different bank quarters.
template <int COLS>
struct TLayout {
  static_assert(COLS % 64 == 0 && COLS <= 512, "COLS must be 64..512, multiple of 64");
  static constexpr int PPR = COLS / 8;          // pieces per k-row
  static constexpr int RPC = 64 / PPR;          // k-rows per deposit
  static constexpr int NCH = kBK / RPC / 4;     // deposits per wave per stage
  static_assert(NCH >= 1, "tile too narrow");
  static constexpr int LDS_ELEMS = kBK * COLS;

  // k-row and logical column (multiple of 8) fetched by this lane in deposit j
  static __device__ __forceinline__ void lane_piece(int j, int& krow, int& col) {
    const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
    krow = (j * 4 + w) * RPC + l / PPR;
    col = ((l % PPR) ^ (2 * (krow & 3))) * 8;
  }
  static __device__ __forceinline__ bf16* deposit(bf16* stage, int j) {
    return stage + (j * 4 + (threadIdx.x >> 6)) * kChunkElems;
  }
  // 32 columns starting at c0 (multiple of 32), k-step kk (16 k-values)
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int c0, int kk) {
    const int l = threadIdx.x & 63;
    const int krow = kk * 16 + 8 * (l >> 5) + ((l & 15) >> 2);
    const int col = c0 + 16 * ((l & 31) >> 4) + 4 * (l & 3);
    const bf16* p = stage + krow * COLS + (((col >> 3) ^ (2 * (krow & 3))) << 3) + (col & 7);
    const bf16x4 lo = lds_read_tr4(p);
    const bf16x4 hi = lds_read_tr4(p + 4 * COLS);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
};

// k-strided operand with a fixed pitch between k-rows (the expert weights)
template <int COLS>
struct TDma {
  using L = TLayout<COLS>;
  static constexpr int NCH = L::NCH;
  static constexpr int LDS_ELEMS = L::LDS_ELEMS;
  const bf16* ptr[NCH];
  int64_t kstride;

  // colptr(c) -> global pointer to (k=0, tile column c), c a multiple of 8; columns outside
  // the matrix must be clamped by the caller to something readable.
  template <class ColPtr>
  __device__ __forceinline__ void init(ColPtr colptr, int64_t ld) {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      int krow, col;
      L::lane_piece(j, krow, col);
      ptr[j] = colptr(col) + (int64_t)krow * ld;
    }
    kstride = (int64_t)kBK * ld;
  }
  __device__ __forceinline__ void issue(int kt, bf16* stage) {
#pragma unroll
    for (int j = 0; j < NCH; ++j) dma16(ptr[j] + kt * kstride, L::deposit(stage, j));
  }
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int c0, int kk) {
    return L::frag(stage, c0, kk);
  }
};

// k-strided operand whose k-rows are the sorted rows [row_begin,row_end) of one expert,
// optionally gathered through an index; k-rows past row_end read the zero block.
template <int COLS>
struct TGatherDma {
  using L = TLayout<COLS>;
  static constexpr int NCH = L::NCH;
  static constexpr int LDS_ELEMS = L::LDS_ELEMS;
  const bf16* mat;
  int64_t ld;
  const int32_t* gather;
  int row_begin, row_end;
  int krow[NCH], col[NCH];
  int32_t rowid[NCH];

  __device__ __forceinline__ void fetch_rows(int kt) {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int rr = row_begin + kt * kBK + krow[j];
      int32_t id = -1;
      if (rr < row_end) id = gather ? gather[rr] : rr;
      rowid[j] = id;
    }
  }
  // columns [col0, col0+COLS) of the matrix; columns >= ncols are clamped to column 0
  __device__ __forceinline__ void init(const bf16* mat_, int64_t ld_, const int32_t* gather_,
                                       int col0, int ncols, int rb, int re) {
    mat = mat_;
    ld = ld_;
    gather = gather_;
    row_begin = rb;
    row_end = re;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      int c;
      L::lane_piece(j, krow[j], c);
      col[j] = col0 + c < ncols ? col0 + c : 0;
    }
    fetch_rows(0);
  }
  // must be called with kt = 0, 1, 2, ... in order: uses the row ids fetched for kt and
  // starts fetching those of kt+1 before the deposits are issued
  __device__ __forceinline__ void issue(int kt, bf16* stage) {
    int32_t cur[NCH];
#pragma unroll
    for (int j = 0; j < NCH; ++j) cur[j] = rowid[j];
    fetch_rows(kt + 1);
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const bf16* src = cur[j] >= 0 ? mat + (int64_t)cur[j] * ld + col[j] : zero_chunk();
      dma16(src, L::deposit(stage, j));
    }
  }
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int c0, int kk) {
    return L::frag(stage, c0, kk);
  }
};

// acc[fn][fm] += Bfrag[fn] x Afrag[fm] over `ktiles` (>= 1) stages of kBK.
// `m_org[fm]` / `n_org[fn]` are the LDS row (or column) origins of this wave's 32-wide
// fragments inside the A / B stage.  On return other waves may still be reading LDS:
// barrier before reusing it.
template <class AOp, class BOp, int FM, int FN>
__device__ __forceinline__ void gemm_mainloop(AOp& A, BOp& B, f32x16 (&acc)[FN][FM], int ktiles,
                                              bf16* lds, const int (&m_org)[FM],
                                              const int (&n_org)[FN]) {
  constexpr int STAGE = AOp::LDS_ELEMS + BOp::LDS_ELEMS;
  constexpr int LOADS = AOp::NCH + BOp::NCH;  // deposits per wave per stage
  constexpr int KK = kBK / 16;
  A.issue(0, lds);
  B.issue(0, lds + AOp::LDS_ELEMS);
  if (ktiles > 1) {
    A.issue(1, lds + STAGE);
    B.issue(1, lds + STAGE + AOp::LDS_ELEMS);
  }
  int stage = 0;
  for (int kt = 0; kt < ktiles; ++kt) {
    // stage kt of every wave has landed; everyone is done reading stage kt-1
    if (kt + 1 < ktiles) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    const bf16* la = lds + stage * STAGE;
    const bf16* lb = la + AOp::LDS_ELEMS;
    bf16x8 af[KK][FM], bf[KK][FN];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int i = 0; i < FM; ++i) af[kk][i] = AOp::frag(la, m_org[i], kk);
#pragma unroll
      for (int j = 0; j < FN; ++j) bf[kk][j] = BOp::frag(lb, n_org[j], kk);
    }
    if (kt + 2 < ktiles) {
      bf16* nx = lds + (stage == 0 ? 2 : stage - 1) * STAGE;
      A.issue(kt + 2, nx);
      B.issue(kt + 2, nx + AOp::LDS_ELEMS);
    }
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int i = 0; i < FM; ++i) acc[j][i] = mfma32(bf[kk][j], af[kk][i], acc[j][i]);
    stage = stage == kStages - 1 ? 0 : stage + 1;
  }
}

// the workgroup's dynamic LDS (size given at launch)
__device__ __forceinline__ bf16* dyn_lds() {
  extern __shared__ __attribute__((aligned(1024))) bf16 momoe_lds[];
  return momoe_lds;
}

template <class AOp, class BOp>
constexpr size_t gemm_lds_bytes() {
  return (size_t)kStages * (AOp::LDS_ELEMS + BOp::LDS_ELEMS) * sizeof(bf16);
}

// Kernels use more than the 64 KiB of LDS a launch gets by default: raise the limit once.
template <class Kernel>
inline void allow_lds(Kernel kernel, size_t bytes, std::once_flag& once) {
  std::call_once(once, [&] {
    (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)bytes);
  });
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
