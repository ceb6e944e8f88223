// Workgroup-level bf16 GEMM building blocks for gfx950 (CDNA4).
//
// A workgroup of 8 wavefronts (two per SIMD: a lone wave leaves ~15% of the MFMA
// issue slots empty) computes a 256 x 256 or, where registers and LDS allow, a 320 x 256 fp32
// tile with v_mfma_f32_32x32x16_bf16; each wave owns 128 x 64 (160 x 64) of it in 8 (10)
// accumulator fragments of 16 registers, one workgroup per CU.  Both MFMA inputs want, per lane, 8
// consecutive k-values of one row (lane%32 = row, lane/32 = which group of 8
// k's).  Two kinds of operand tile feed that:
//
//   RDma  - "k-contiguous": the operand is stored [row][k] in global memory.
//           LDS stage [ROWS][32]; a fragment is one ds_read_b128.
//   TDma  - "k-strided": the operand is stored [k][col] (the layout of the
//           expert weights in the forward GEMMs, and of everything in the
//           weight-gradient GEMMs).  LDS stage [32][256]; a fragment is two
//           ds_read_b64_tr_b16, the gfx950 LDS transpose read: within each
//           group of 16 lanes, lane i supplies the address of 4 consecutive
//           columns of k-row i/4 (columns 4*(i%4)..+3) and receives column i
//           of those 4 k-rows.
//
// Sizing facts measured on MI355X that shape this file:
//   * Under sustained MFMA load the chip is power-limited: a loop of nothing but this MFMA on
//     random operands runs at 1.75 PFLOP/s with the shader clock at 1.73 GHz (2.3 PFLOP/s at
//     2.4 GHz on zeros), the complete main loop at 1.6-1.7 GHz.  Time then follows the energy
//     spent - multiplications, LDS and L2 traffic - far more than exposed latencies: useless
//     work costs, idle cycles barely do.
//   * LDS serves 16 lanes per clock: 256 B/clk for bank-conflict-free
//     ds_read_b128, 128 B/clk at best for the transpose reads.
//   * A CU streams at most ~27 B/clk from L2 and ~19 B/clk from beyond it, and tile
//     traffic of this shape sustains ~19 B/clk (11.7 TB/s over the chip), which a 256x256 tile
//     - the largest the register file holds - needs at ~60% of the MFMA peak: the loads
//     set the pace as much as the MFMA pipe, and several stages must be in flight at all times.
//   * The transfer instruction must take "uniform base + 32-bit lane offset": with a 64-bit
//     address per lane a whole GEMM ran 20% slower.
//   * Launching one 256x256 tile per workgroup costs ~25% in launch, pipeline fill
//     and drain: workgroups are persistent and prefetch across tiles.
//   * Rows of a ragged tile that do not exist are pointed at the last valid row: the 16
//     lanes of a deposit then ask for one line instead of 16.  What a small tile cannot avoid
//     is streaming its whole weight block, so an expert's rows are cut into equal row tiles
//     rather than full tiles plus a sliver, and a taller tile saves whole passes over the weights:
//     with 320-row tiles an expert of 513..640 rows takes two passes instead of three (measured
//     -9..-11% for such experts, -10% of the bytes per flop for large ones).
//
// Global memory goes straight to LDS with global_load_lds_dwordx4 (no VGPR
// staging): one wave instruction deposits 64 x 16 bytes contiguously.  Since
// every lane chooses its own global address, the LDS image is swizzled by
// permuting WHICH 16-byte piece each lane fetches: rows keep their natural,
// unpadded pitch, and the fragment reads above are bank-conflict free.  The same
// freedom does all predication: a lane that would read outside the matrix is
// pointed at a clamped row/column (results masked at the store; along k the main loop
// zeroes the affected fragment registers instead).
//
// The k-loop runs a ring of 3 or 4 stages of 32 k: while one stage is multiplied (2 MFMA
// k-steps) the next two or three are in flight; one s_barrier per stage.  The fragments of
// a stage's second k-step are read before the barrier that opens the next stage and
// multiplied after it, so the matrix pipe stays fed while the first fragments of
// the new stage travel from LDS.  At the end of a tile all buffers but one are free, so
// the next tile's first stages are requested before the epilogue starts.
//
// The MFMA is issued with the N-side fragment as its first input and the M-side
// fragment as its second, so each lane ends up holding, for ONE tile row
// (lane%32), groups of 4 consecutive columns: register r of the 16 holds
// column 8*(r/4) + 4*(lane/32) + r%4.  Row-wise epilogues (per-row scale,
// SwiGLU pairing, row reductions) are then lane-local and stores are 8-byte.
#pragma once
#include <atomic>
#include <mutex>

#include "common.hpp"

namespace momoe {

constexpr int kBK = 32;            // k-extent of one LDS stage
constexpr int kKSteps = kBK / 16;  // MFMA k-steps per stage
constexpr int kChunkElems = 512;   // one wave-wide 16-byte-per-lane deposit = 1 KiB

// 16 bytes per lane, global -> LDS.  `lds_wave_base` is a wave-uniform LDS byte address; lane
// L's bytes land at lds_wave_base + 16*L.  Completion is tracked by vmcnt.  Issued as inline
// assembly so that the compiler's own wait-count insertion does not know about the
// transfer: with the builtin it forces vmcnt(0) in front of the LDS transpose reads.
// Ordering is therefore entirely manual: wait_vmcnt<>() + s_barrier before a stage is
// read, s_barrier before it is overwritten.
// LDS byte address of a pointer into LDS (done once per kernel; transfers then use integers)
__device__ __forceinline__ uint32_t lds_address(bf16* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) bf16*)p;
}
__device__ __forceinline__ void dma16(const bf16* g, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g),
               "s"(__builtin_amdgcn_readfirstlane(lds_wave_base))
               : "memory");
}
// same, the source given as a wave-uniform base plus a per-lane byte offset
__device__ __forceinline__ void dma16(const bf16* uniform_base, uint32_t byte_offset,
                                      uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(byte_offset),
               "s"(uniform_base), "s"(__builtin_amdgcn_readfirstlane(lds_wave_base))
               : "memory");
}

// wait until at most N vector-memory operations of this wave are outstanding
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}
// wait until every LDS / scalar-memory operation of this wave has returned
__device__ __forceinline__ void wait_lgkm0() { __builtin_amdgcn_s_waitcnt(0xC07F); }

__device__ __forceinline__ bf16x4 lds_read_tr4(const bf16* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4 __attribute__((address_space(3)))*)p);
}

__device__ __forceinline__ f32x16 mfma32(bf16x8 first, bf16x8 second, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(first, second, c, 0, 0, 0);
}

// uniform (scalar-unit) load of an int32 that no kernel writes while this one runs
__device__ __forceinline__ int32_t load_uniform(const int32_t* p) {
  return *(const int32_t __attribute__((address_space(4)))*)p;
}

// ---- k-contiguous operand -------------------------------------------------------------
// LDS stage: row r at elements [32r, 32r+32); its four 16-byte k-pieces are stored at
// position piece ^ ((r>>2)&3), so the 16 rows x 16 bytes that 16 consecutive lanes of a
// fragment read touch cover 16 different 16-byte bank groups (256 bytes, one clock).
template <int ROWS>
struct RDma {
  static_assert(ROWS % (16 * kWaves) == 0, "ROWS must be a multiple of 16 rows per wave");
  static constexpr int NCH = ROWS / (16 * kWaves);  // deposits per wave per stage (16 rows each)
  static constexpr int LDS_ELEMS = ROWS * kBK;
  const bf16* base;   // wave-uniform
  uint32_t off[NCH];  // byte offset of this lane's piece of deposit j from `base`, at k=0

  // tile row whose piece this lane fetches in deposit j
  static __device__ __forceinline__ int row_of(int j) {
    return (j * kWaves + wave_id()) * 16 + ((threadIdx.x & 63) >> 2);
  }
  // row r of the tile starts at (char*)base_ + rowoff(r, j), j being the deposit that fetches
  // it for this lane (r = row_of(j)); every r < ROWS must be readable
  template <class RowOff>
  __device__ __forceinline__ void init(const bf16* base_, RowOff rowoff) {
    const int l = threadIdx.x & 63;
    base = base_;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int row = row_of(j);
      const int piece = (l & 3) ^ ((row >> 2) & 3);
      off[j] = rowoff(row, j) + piece * 16;
    }
  }
  __device__ __forceinline__ void issue(int kt, uint32_t stage) {
    const int w = wave_id();
    const bf16* b = base + kt * kBK;
#pragma unroll
    for (int j = 0; j < NCH; ++j) dma16(b, off[j], stage + (j * kWaves + w) * (kChunkElems * 2));
  }
  template <int S>
  __device__ __forceinline__ void issue_head(uint32_t stage) { issue(S, stage); }
  // 32 rows starting at r0 (multiple of 32), k-step kk (16 k-values)
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int r0, int kk) {
    const int l = threadIdx.x & 63;
    const int row = r0 + (l & 31);
    const int piece = (2 * kk + (l >> 5)) ^ ((row >> 2) & 3);
    return *(const bf16x8*)(stage + row * kBK + piece * 8);
  }
};

// The same LDS stage fed from a k-blocked matrix: element (row, k) at
// mat[((k / 32) * nrows + row) * 32 + k % 32].  Intermediates that this library both writes and
// reads (h between the two forward GEMMs) are stored like this: a stage of consecutive rows is
// one contiguous block of memory, fetched in whole 128-byte lines, where the row-major layout
// asks for half a line per row and stage.
template <int ROWS>
struct RBlockedDma {
  using R = RDma<ROWS>;
  static constexpr int NCH = R::NCH;
  static constexpr int LDS_ELEMS = R::LDS_ELEMS;
  R r;
  int64_t kstride;  // elements between consecutive k-blocks = 32 * rows of the matrix
  // rows [row0, row0 + ROWS) of the matrix; rows >= nvalid (tile-local) are clamped to the last
  __device__ __forceinline__ void init(const bf16* mat, int64_t nrows, int64_t row0, int nvalid) {
    kstride = nrows * kBK;
    r.init(mat + row0 * kBK, [&](int row, int) { return (uint32_t)min(row, nvalid - 1) * (uint32_t)(kBK * 2); });
  }
  __device__ __forceinline__ void issue(int kt, uint32_t stage) {
    const int w = wave_id();
    const bf16* b = r.base + (int64_t)kt * kstride;
#pragma unroll
    for (int j = 0; j < NCH; ++j) dma16(b, r.off[j], stage + (j * kWaves + w) * (kChunkElems * 2));
  }
  template <int S>
  __device__ __forceinline__ void issue_head(uint32_t stage) { issue(S, stage); }
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int r0, int kk) { return R::frag(stage, r0, kk); }
};

// ---- k-strided operand, 256 columns -----------------------------------------------------
// LDS stage: k-row k at elements [256k, 256k+256); 16-byte piece p of the row is stored
// at position p ^ swz(k), swz(k) = 4*(k&3) + 16*((k>>3)&1): the 8 k-rows x 64 bytes that one
// transpose read of a wave touches then fall into 8 different 64-byte bank groups (measured
// 124 B/clk against 113 for a swizzle that only separates the 4 k-rows of a 16-lane group;
// the instruction tops out at 128).  A deposit covers two k-rows (lanes 0-31 / 32-63); wave w
// deposits k-rows [4w, 4w+4).
struct TLayout {
  static constexpr int COLS = 256;
  static constexpr int NCH = kBK / (2 * kWaves);  // deposits per wave per stage
  static constexpr int LDS_ELEMS = kBK * COLS;
  static __device__ __forceinline__ int swz(int krow) { return 4 * (krow & 3) + 16 * ((krow >> 3) & 1); }

  // k-row and logical column (multiple of 8) fetched by this lane in deposit j
  static __device__ __forceinline__ void lane_piece(int j, int& krow, int& col) {
    const int l = threadIdx.x & 63, w = wave_id();
    krow = w * (2 * NCH) + j * 2 + (l >> 5);
    col = ((l & 31) ^ swz(krow)) * 8;
  }
  static __device__ __forceinline__ uint32_t deposit(uint32_t stage, int j) {
    return stage + (wave_id() * NCH + j) * (kChunkElems * 2);
  }
  // 32 columns starting at c0 (multiple of 32), k-step kk (16 k-values)
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int c0, int kk) {
    const int l = threadIdx.x & 63;
    const int krow = kk * 16 + 8 * (l >> 5) + ((l & 15) >> 2);
    const int col = c0 + 16 * ((l & 31) >> 4) + 4 * (l & 3);
    // k-rows krow and krow+4 share the swizzle, so the second read is a fixed distance away
    const bf16* p = stage + krow * COLS + (((col >> 3) ^ swz(krow)) << 3) + (col & 7);
    const bf16x4 lo = lds_read_tr4(p);
    const bf16x4 hi = lds_read_tr4(p + 4 * COLS);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
};

// k-strided operand with a fixed pitch between k-rows (the expert weights)
struct TDma {
  using L = TLayout;
  static constexpr int NCH = L::NCH;
  static constexpr int LDS_ELEMS = L::LDS_ELEMS;
  const bf16* base;   // wave-uniform
  uint32_t off[NCH];  // byte offset of this lane's piece of deposit j from `base`, at k=0
  int64_t kstride;

  // coloff(c) -> element offset from base_ of (k=0, tile column c), c a multiple of 8;
  // columns outside the matrix must be clamped by the caller to something readable.
  // ld = elements between consecutive k-rows.
  template <class ColOff>
  __device__ __forceinline__ void init(const bf16* base_, ColOff coloff, int64_t ld) {
    base = base_;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      int krow, col;
      L::lane_piece(j, krow, col);
      off[j] = (uint32_t)((coloff(col) + (int64_t)krow * ld) * 2);
    }
    kstride = (int64_t)kBK * ld;
  }
  __device__ __forceinline__ void issue(int kt, uint32_t stage) {
    const bf16* b = base + kt * kstride;
#pragma unroll
    for (int j = 0; j < NCH; ++j) dma16(b, off[j], L::deposit(stage, j));
  }
  template <int S>
  __device__ __forceinline__ void issue_head(uint32_t stage) { issue(S, stage); }
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int c0, int kk) {
    return L::frag(stage, c0, kk);
  }
};

// k-strided operand whose k-rows are the sorted rows [row_begin,row_end) of one expert,
// optionally gathered through an index.  k-rows past row_end are pointed at the expert's last
// row (any readable row would do): the main loop zeroes the M-side fragments of those k-values
// in the last stage, so they add nothing.  The four row ids of a wave's deposits are
// wave-uniform and come through scalar loads: those of the first NFIRST stages once per expert
// (every tile of the expert starts with the same rows), the later ones one stage ahead of their
// use.  Asking for the ids (request) and turning them into offsets (resolve) are separate steps
// a stage apart: done in one step, every wave sat out one scalar-load latency per stage right
// after the barrier, before its transfers went out.  Sources are given as a wave-uniform base
// plus a 32-bit byte offset per lane (the form with a full 64-bit address per lane costs ~20% of
// the whole GEMM): the base is the matrix for a gathered operand and the expert's first row
// otherwise, so (number of tokens) x (row pitch) must stay below 4 GiB.
// MAY_GATHER = false: the rows are never gathered and no ids are loaded.  NFIRST = stages of a
// tile that are requested ahead of its main loop (the depth of the ring it is used with, less one).
template <bool MAY_GATHER, int NFIRST>
struct TGatherDmaT {
  using L = TLayout;
  static constexpr int NCH = L::NCH;
  static constexpr int LDS_ELEMS = L::LDS_ELEMS;
  static constexpr int kRows = 2 * NCH;  // k-rows of one wave's deposits in a stage
  static_assert(NCH == 2, "a wave's deposits of one stage cover four consecutive rows");
  const bf16* mat;  // wave-uniform
  uint32_t ldb;     // bytes between rows
  const int32_t* gather;
  int row_begin, row_end;
  uint32_t colb[NCH];  // byte offset of this lane's columns in deposit j
  struct Offs {
    uint32_t a[NCH], b[NCH];  // byte offsets of the two k-rows of each deposit
  };
  struct Ids {
    int32_t v[kRows];
  };
  Offs head[NFIRST];  // this wave's k-rows in the first stages of a tile
  Ids next;           // ids requested for the next issue() call

  // sorted row behind k-row j of this wave's deposits in stage kt
  __device__ __forceinline__ int row_of(int kt, int j) const {
    const int w = wave_id();
    return min(row_begin + kt * kBK + w * kRows + j, row_end - 1);
  }
  // start the scalar loads of the ids of stage kt; the results must not be touched before
  // resolve()
  __device__ __forceinline__ void request(int kt, Ids& ids) const {
    if (!MAY_GATHER || gather == nullptr) return;  // kernel-uniform
#pragma unroll
    for (int j = 0; j < kRows; ++j) ids.v[j] = load_uniform(gather + row_of(kt, j));
  }
  __device__ __forceinline__ Offs resolve(int kt, const Ids& ids) const {
    uint32_t o[kRows];
#pragma unroll
    for (int j = 0; j < kRows; ++j)
      o[j] = (uint32_t)(MAY_GATHER && gather != nullptr ? ids.v[j] : row_of(kt, j) - row_begin) * ldb;
    Offs out;
#pragma unroll
    for (int j = 0; j < NCH; ++j) out.a[j] = o[2 * j], out.b[j] = o[2 * j + 1];
    return out;
  }
  // once per expert (re > rb); ld_ = elements between rows of the matrix
  __device__ __forceinline__ void set_rows(const int32_t* gather_, int64_t ld_, int rb, int re) {
    gather = gather_;
    ldb = (uint32_t)(ld_ * 2);
    row_begin = rb;
    row_end = re;
    Ids first[NFIRST];  // all in flight before the first is used
#pragma unroll
    for (int s = 0; s < NFIRST; ++s) request(s, first[s]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < NFIRST; ++s) head[s] = resolve(s, first[s]);
  }
  // per tile: columns [col0, col0+256) of the matrix; columns >= ncols are clamped to column 0
  __device__ __forceinline__ void set_cols(const bf16* mat_, int col0, int ncols) {
    mat = gather ? mat_ : (const bf16*)((const char*)mat_ + (int64_t)row_begin * ldb);
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      int krow, c;
      L::lane_piece(j, krow, c);
      colb[j] = (uint32_t)(col0 + c < ncols ? col0 + c : 0) * 2;
    }
  }
  __device__ __forceinline__ void deposit(const Offs v, uint32_t stage) const {
    const bool upper = (threadIdx.x & 63) >= 32;
#pragma unroll
    for (int j = 0; j < NCH; ++j)
      dma16(mat, (upper ? v.b[j] : v.a[j]) + colb[j], L::deposit(stage, j));
  }
  // stage S < NFIRST of a tile; the last of them asks for the ids of issue(NFIRST)
  template <int S>
  __device__ __forceinline__ void issue_head(uint32_t stage) {
    static_assert(S < NFIRST, "only the first stages are cached");
    deposit(head[S], stage);
    if (S == NFIRST - 1) request(NFIRST, next);
  }
  // must be called with kt = NFIRST, NFIRST+1, ... in order: uses the ids requested for kt (a
  // stage ago: they have long arrived) and asks for those of kt+1 only after that
  __device__ __forceinline__ void issue(int kt, uint32_t stage) {
    const Offs cur = resolve(kt, next);
    __builtin_amdgcn_sched_barrier(0);
    request(kt + 1, next);
    deposit(cur, stage);
  }
  static __device__ __forceinline__ bf16x8 frag(const bf16* stage, int c0, int kk) {
    return L::frag(stage, c0, kk);
  }
};
// ---- the k-loop -----------------------------------------------------------------------------
// Ring of NS LDS stage buffers; `head` is the buffer of stage 0 of the current tile and is
// carried from tile to tile by a persistent workgroup.  FIRST = NS - 1 stages of a tile are
// requested ahead of its main loop (during the previous tile's epilogue).  Every kernel here uses
// four buffers: with three, the GEMMs whose weights stream k-row by k-row from HBM ran 3-7 % slower
// (two stages in flight do not cover that latency); the others did not care.
template <class AOp, class BOp, int NS>
struct StageRing {
  static_assert(NS >= 3 && NS <= 5, "ring depth");
  using A = AOp;
  using B = BOp;
  static constexpr int STAGES = NS, FIRST = NS - 1;
  static constexpr int STAGE = AOp::LDS_ELEMS + BOp::LDS_ELEMS;
  static constexpr size_t BYTES = (size_t)NS * STAGE * sizeof(bf16);
  bf16* lds;
  uint32_t addr;  // LDS byte address of `lds`
  int head;
  __device__ __forceinline__ explicit StageRing(bf16* lds_) : lds(lds_), addr(lds_address(lds_)), head(0) {}
  static __device__ __forceinline__ int slot(int s) {
    return (NS & (NS - 1)) == 0 ? s & (NS - 1) : (int)((unsigned)s % (unsigned)NS);
  }
  __device__ __forceinline__ bf16* buf(int kt) const { return lds + slot(kt + head) * STAGE; }
  __device__ __forceinline__ uint32_t buf_addr(int kt) const {
    return addr + slot(kt + head) * (STAGE * 2);
  }
  __device__ __forceinline__ void advance(int ktiles) { head = slot(head + ktiles); }
  // After a tile's main loop (the ring has advanced): the one buffer that the next tile's first
  // stages do not use, i.e. the finished tile's last stage.  Free for the epilogue once every
  // wave has left the main loop (a barrier), until the next main loop's first barrier.
  __device__ __forceinline__ bf16* free_buf() const { return lds + slot(head + FIRST) * STAGE; }
};

template <class AOp, class BOp, int NS>
__device__ __forceinline__ void gemm_issue(AOp& A, BOp& B, StageRing<AOp, BOp, NS>& ring, int kt) {
  const uint32_t st = ring.buf_addr(kt);
  A.issue(kt, st);
  B.issue(kt, st + AOp::LDS_ELEMS * 2);
}

// Request the first stages of a tile.  May be called right after the previous tile's
// main loop, while other waves still multiply its last stage: the other buffers were
// released by that tile's last barrier.
template <int S, class AOp, class BOp, int NS>
__device__ __forceinline__ void gemm_issue_head(AOp& A, BOp& B, StageRing<AOp, BOp, NS>& ring) {
  const uint32_t st = ring.buf_addr(S);
  A.template issue_head<S>(st);
  B.template issue_head<S>(st + AOp::LDS_ELEMS * 2);
}
template <class AOp, class BOp, int NS>
__device__ __forceinline__ void gemm_issue_first(AOp& A, BOp& B, StageRing<AOp, BOp, NS>& ring,
                                                 int ktiles) {
  constexpr int kFirst = NS - 1;
  gemm_issue_head<0>(A, B, ring);
  if (ktiles > 1) gemm_issue_head<1>(A, B, ring);
  if constexpr (kFirst > 2) {
    if (ktiles > 2) gemm_issue_head<2>(A, B, ring);
  }
  if constexpr (kFirst > 3) {
    if (ktiles > 3) gemm_issue_head<3>(A, B, ring);
  }
}

// Waits on the transfers count operations: loads of a wave complete in the order they were
// issued, so "at most n outstanding" means "all loads but the youngest n are done" (stores that
// are still in flight only make the wait longer).  Each wait allows exactly the stages known
// to have been requested after the one that is needed.
template <int LOADS, int kFirst>
__device__ __forceinline__ void wait_first_stage(int ktiles) {
  static_assert((kFirst - 1) * LOADS <= 63, "vmcnt is a 6-bit counter");
  static_assert(kFirst >= 2 && kFirst <= 4, "wait ladder written for 2 to 4 stages ahead");
  if (kFirst >= 4 && ktiles > 3) wait_vmcnt<3 * LOADS>();
  else if (kFirst >= 3 && ktiles > 2) wait_vmcnt<2 * LOADS>();
  else if (ktiles > 1) wait_vmcnt<LOADS>();
  else wait_vmcnt<0>();
}
// wait until the deposits of stage kt (>= 1) have landed, when the stages up to kt+kStages-2
// have been requested and everything older than stage kt is known to be complete
template <int LOADS, int kStages>
__device__ __forceinline__ void wait_stage(int kt, int ktiles) {
  static_assert((kStages - 2) * LOADS <= 63, "vmcnt is a 6-bit counter");
  static_assert(kStages >= 3 && kStages <= 5, "wait ladder written for 3 to 5 stages");
  if (kStages >= 5 && kt + 3 < ktiles) wait_vmcnt<3 * LOADS>();
  else if (kStages >= 4 && kt + 2 < ktiles) wait_vmcnt<2 * LOADS>();
  else if (kt + 1 < ktiles) wait_vmcnt<LOADS>();
  else wait_vmcnt<0>();
}

// acc[fn][fm] += Bfrag[fn] x Afrag[fm] over `ktiles` (>= 1) stages of kBK.  The first stages
// must already have been requested with gemm_issue_first.  NA is the number of 32-row
// fragment rows of this wave that hold valid rows (wave-uniform): the others are neither read
// nor multiplied; with NA = 0 the wave only takes part in the transfers and barriers.
// `ktail` (1..kBK) is the number of k-values of the last stage that exist.
// `hook` runs once, right after the barrier that opens the tile: loads issued there travel
// under the whole main loop (they enter the vmcnt queue between two stages, which can only
// make the stage waits err on the long side).  On return the ring has advanced to the next
// tile; all buffers but the last stage's are free, other waves may still be reading that one.
template <class AOp, class BOp, int NS, int FM, int FN, int NA, class Hook>
__device__ __forceinline__ void gemm_mainloop(AOp& A, BOp& B, f32x16 (&acc)[FN][FM], int ktiles,
                                              StageRing<AOp, BOp, NS>& ring, const int (&m_org)[FM],
                                              const int (&n_org)[FN], Hook hook, int ktail = kBK) {
  constexpr int kStages = NS, kFirst = NS - 1;
  static_assert(kKSteps == 2, "written for 2 k-steps per stage");
  static_assert(NA >= 0 && NA <= FM, "active fragment rows");
  constexpr int LOADS = AOp::NCH + BOp::NCH;
  bf16x8 af[2][FM], bf[2][FN];
  auto load_frags = [&](int kt, int kk) {
    if (NA == 0) return;
    const bf16* la = ring.buf(kt);
    const bf16* lb = la + AOp::LDS_ELEMS;
#pragma unroll
    for (int i = 0; i < NA; ++i) af[kk][i] = AOp::frag(la, m_org[i], kk);
#pragma unroll
    for (int j = 0; j < FN; ++j) bf[kk][j] = BOp::frag(lb, n_org[j], kk);
  };
  auto multiply = [&](int kk) {
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int i = 0; i < NA; ++i) acc[j][i] = mfma32(bf[kk][j], af[kk][i], acc[j][i]);
  };
  // The scheduling fences keep the compiler from hoisting fragment reads across k-steps.
  auto fence = [] { __builtin_amdgcn_sched_barrier(0); };

  // Stage 0 has landed (the previous tile's stores need not have); every wave is done reading
  // the previous tile, whose last buffer the next stage will reuse.
  wait_first_stage<LOADS, kFirst>(ktiles);
  wait_lgkm0();
  __builtin_amdgcn_s_barrier();
  fence();
#pragma unroll
  for (int s = kFirst; s < kStages; ++s)
    if (ktiles > s) gemm_issue(A, B, ring, s);
  hook();
  fence();
  load_frags(0, 0);
  fence();
  // the last stage is peeled off so that the loop body has a single path: a branch around
  // the barrier would make the compiler wait for the freshly issued fragment reads
  for (int kt = 0; kt + 1 < ktiles; ++kt) {
    load_frags(kt, 1);
    multiply(0);
    fence();
    // stage kt+1 has landed; all LDS reads of stage kt have returned, so its buffer may be
    // overwritten once every wave is past the barrier
    wait_stage<LOADS, kStages>(kt + 1, ktiles);
    wait_lgkm0();
    __builtin_amdgcn_s_barrier();
    fence();
    if (kt + kStages < ktiles) gemm_issue(A, B, ring, kt + kStages);
    fence();
    load_frags(kt + 1, 0);
    multiply(1);
    fence();
  }
  load_frags(ktiles - 1, 1);
  if (ktail < kBK) {
    // only the first `ktail` k-values of the last stage exist: zero the rest on the M side
    // (a lane holds k-values 16*kk + 8*(lane/32) + 0..7 of its row, two per register)
    wait_lgkm0();
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) {
      const int nvalid = ktail - 16 * kk - 8 * (int)((threadIdx.x & 63) >> 5);
#pragma unroll
      for (int i = 0; i < NA; ++i) {
        u32x4 v = __builtin_bit_cast(u32x4, af[kk][i]);
#pragma unroll
        for (int d = 0; d < 4; ++d)
          v[d] &= nvalid >= 2 * d + 2 ? 0xFFFFFFFFu : nvalid == 2 * d + 1 ? 0x0000FFFFu : 0u;
        af[kk][i] = __builtin_bit_cast(bf16x8, v);
      }
    }
  }
  multiply(0);
  fence();
  multiply(1);
  fence();
  ring.advance(ktiles);
}

// Row-tile geometry of a kernel: two wave rows of FM 32-row fragment rows each (tiles of up to
// 64 * FM rows, 64 columns per wave), the rows of the row operand's stage buffer (whole deposits
// of 16 rows per wave, so a multiple of 128 that holds the tallest tile) and the ring depth.
template <int FM_, int NS_>
struct RowTileGeometry {
  static constexpr int FM = FM_, FN = 2;
  static constexpr int MAX_ROWS = 64 * FM;
  static constexpr int AROWS = (MAX_ROWS + 127) / 128 * 128;
  static constexpr int STAGES = NS_;
};
// 256-row tiles: the recomputing GEMM, whose epilogue leaves no registers for more, and any
// launch whose tile table holds no taller tile (a routing in which no expert has more than 256
// rows gains nothing from tall tiles and pays for their third deposit per stage and their
// register pressure: a 16-token decode call ran 10% slower on them)
using StdTiles = RowTileGeometry<4, 4>;
// 320-row tiles: 10 accumulator fragments per wave and a 384-row stage buffer whose last 64 rows
// repeat the tile's last row; four such stages are all of the CU's LDS (the epilogues stage
// their stores in the ring's idle buffer)
using TallTiles = RowTileGeometry<5, 4>;
static_assert(TallTiles::MAX_ROWS == MOMOE_TILE_ROWS && StdTiles::MAX_ROWS == MOMOE_RECOMPUTE_TILE_ROWS,
              "tile heights promised by the header");

// main loop for a wave that owns `na` fragment rows starting at tile row m_org[0]
template <class AOp, class BOp, int NS, int FM, int FN, class Hook>
__device__ __forceinline__ void gemm_rows(AOp& A, BOp& B, f32x16 (&acc)[FN][FM], int ktiles,
                                          StageRing<AOp, BOp, NS>& ring, const int (&m_org)[FM],
                                          const int (&n_org)[FN], int na_, Hook hook) {
  static_assert(FM == 4 || FM == 5, "dispatch written for 4 or 5 fragment rows per wave");
  const int na = __builtin_amdgcn_readfirstlane(na_);
  if constexpr (FM == 5) {
    if (na == 5) {
      gemm_mainloop<AOp, BOp, NS, FM, FN, 5>(A, B, acc, ktiles, ring, m_org, n_org, hook);
      return;
    }
  }
  if (na == 4) gemm_mainloop<AOp, BOp, NS, FM, FN, 4>(A, B, acc, ktiles, ring, m_org, n_org, hook);
  else if (na == 3) gemm_mainloop<AOp, BOp, NS, FM, FN, 3>(A, B, acc, ktiles, ring, m_org, n_org, hook);
  else if (na == 2) gemm_mainloop<AOp, BOp, NS, FM, FN, 2>(A, B, acc, ktiles, ring, m_org, n_org, hook);
  else if (na == 1) gemm_mainloop<AOp, BOp, NS, FM, FN, 1>(A, B, acc, ktiles, ring, m_org, n_org, hook);
  else gemm_mainloop<AOp, BOp, NS, FM, FN, 0>(A, B, acc, ktiles, ring, m_org, n_org, hook);
}

// the workgroup's dynamic LDS (size given at launch)
__device__ __forceinline__ bf16* dyn_lds() {
  extern __shared__ __attribute__((aligned(1024))) bf16 momoe_lds[];
  return momoe_lds;
}

// Kernels use more than the 64 KiB of LDS a launch gets by default: the limit is raised once per
// kernel, and the outcome kept, so that an entry point whose kernel cannot have its LDS reports
// it instead of failing at every launch for no visible reason.
struct LdsLimit {
  std::once_flag once;
  bool ok = false;
};
template <class Kernel>
inline bool allow_lds(Kernel kernel, size_t bytes, LdsLimit& lim) {
  std::call_once(lim.once, [&] {
    lim.ok = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                 (int)bytes) == hipSuccess;
    if (!lim.ok) (void)hipGetLastError();
  });
  return lim.ok;
}

// number of persistent workgroups: one per CU of the current device, rounded to the 8 XCDs
// (the CU count of a device is looked up once)
inline int persistent_grid() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    cached[dev].store(cus, std::memory_order_relaxed);
  }
  return (cus + 7) / 8 * 8;
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

__device__ __forceinline__ bf16x4 pack_bf16x4(float a, float b, float c, float d) {
  return bf16x4{(bf16)a, (bf16)b, (bf16)c, (bf16)d};
}
__device__ __forceinline__ void store_bf16x4(bf16* p, float a, float b, float c, float d) {
  *(bf16x4*)p = pack_bf16x4(a, b, c, d);
}

// LDS the epilogues stage their stores in (RowStager below): 4 KiB per wave
constexpr int kStageBytesPerWave = 32 * 64 * 2;                  // NF = 2
constexpr size_t kEpilogueLds = (size_t)kWaves * kStageBytesPerWave;

// ---- persistent tile loop ------------------------------------------------------------------------
// Drives a workgroup through its (row tile, column block) pairs with everything a tile needs
// from memory requested one tile ahead.  The tile program P supplies
//   typename P::Prep                          per-tile values that come from loads
//   gather(tile, prep)                        issue those loads; must not use their results
//   late(tile, prep)                          loads that depend on gather()'s results: issued
//                                             a tile later, under the tile's own main loop
//   setup(tile, prep, A, B)                   operand set-up (may use gather()'s results)
//   epilogue(tile, acc, prep, staging)        may use late()'s results; staging = kEpilogueLds
//                                             bytes of LDS for the workgroup
//   ktiles                                    stages per tile
// While tile t is multiplied: the table entry of tile t+2 and the gathered values of tile t+1
// are in flight; after its main loop the first stages of tile t+1 are requested, then the
// epilogue of tile t runs.
template <int FM, int FN, class P, class AOp, class BOp, int NS>
__device__ __forceinline__ void run_row_tiles(P& prog, TileSched& sched, StageRing<AOp, BOp, NS>& ring,
                                              const int (&n_org)[FN]) {
  static_assert(StageRing<AOp, BOp, NS>::STAGE * sizeof(bf16) >= kEpilogueLds, "a stage buffer holds the store staging");
  TileCoord c0 = sched.next();
  if (!c0.valid) return;
  TileCoord c1 = sched.next();
  typename P::Prep p0, p1;
  AOp A;
  BOp B;
  prog.gather(c0, p0);
  prog.setup(c0, p0, A, B);
  gemm_issue_first(A, B, ring, prog.ktiles);
  p1 = p0;
  while (true) {
    f32x16 acc[FN][FM];
    zero_acc<FM, FN>(acc);
    TileSched::Raw rn;
    int m_org[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) m_org[i] = c0.mbase + 32 * i;
    gemm_rows<AOp, BOp, NS, FM, FN>(A, B, acc, prog.ktiles, ring, m_org, n_org, c0.na, [&] {
      prog.late(c0, p0);
      if (c1.valid) prog.gather(c1, p1);
      rn = sched.fetch();
    });
    if (c1.valid) {
      prog.setup(c1, p1, A, B);
      gemm_issue_first(A, B, ring, prog.ktiles);  // travels during this tile's epilogue
    }
    // the epilogue stages its stores in the ring's idle buffer: every wave must have read the
    // last stage out of it
    wait_lgkm0();
    __builtin_amdgcn_s_barrier();
    prog.epilogue(c0, acc, p0, ring.free_buf());
    if (!c1.valid) break;
    c0 = c1;
    p0 = p1;
    c1 = sched.resolve(rn);
  }
}

// ---- coalesced epilogue stores ----------------------------------------------------------------
// In the accumulator layout a lane owns 4 consecutive columns of one row, so a direct store
// writes 8-byte pieces scattered over 32 rows and every 128-byte line is written in 8 partial
// requests.  Instead each wave passes one 32-row fragment row at a time through a private LDS
// area (32 rows x 32*NF columns) and reads it back with 16 bytes per lane, lanes running along
// the rows: stores then cover whole lines.  Wave-private: no barrier is involved.

template <int NF>
struct RowStager {
  static constexpr int CHUNKS = 4 * NF;        // 16-byte chunks per staged row
  static constexpr int PITCH = 32 * NF;        // elements per staged row
  static constexpr int PASSES = 32 * CHUNKS / 64;
  // The 16-byte chunks of a staged row are permuted by the row.  The 64 banks hold 256 bytes, i.e.
  // 256 / (2 * PITCH) consecutive rows, so the permutation changes from one such group of rows to
  // the next: the 32 rows x 8 bytes that a half-wave put()s at a time then spread over the banks.
  // Measured (SQ_LDS_BANK_CONFLICT per launch of the headline layer): with 64-byte rows (NF = 1,
  // the x.Wl1 kernels) a third of what permuting by the row itself gave (3.4 M -> 1.1 M forward,
  // 6.5 M -> 2.2 M backward); with 128-byte rows (NF = 2) no change, 1024 cycles per tile.
  static constexpr int ROWS_PER_BANK_ROW = 256 / (2 * PITCH);
  static __device__ __forceinline__ int swz(int row) { return (row / ROWS_PER_BANK_ROW) & (CHUNKS - 1); }
  bf16* st;  // this wave's staging area

  // `slot` selects one of the 2/NF staging areas of this wave
  __device__ __forceinline__ explicit RowStager(bf16* epilogue_lds, int slot = 0)
      : st(epilogue_lds + wave_id() * (kStageBytesPerWave / 2) + slot * (32 * PITCH)) {}

  // this lane's quad q of fragment f: row lane%32, columns 32f + 8q + 4*(lane/32) .. +3
  __device__ __forceinline__ void put(int f, int q, bf16x4 v) const {
    const int l = threadIdx.x & 63, row = l & 31, half = l >> 5;
    const int c = (4 * f + q) ^ swz(row);
    *(bf16x4*)(st + row * PITCH + c * 8 + half * 4) = v;
  }
  // pass p of PASSES: 16 bytes = columns [col, col+8) of row `row` (both relative to the
  // fragment row: row in [0,32), col in [0, 32*NF))
  __device__ __forceinline__ bf16x8 get(int p, int& row, int& col) const {
    const int l = threadIdx.x & 63;
    row = p * (64 / CHUNKS) + l / CHUNKS;
    const int pc = l % CHUNKS;
    col = (pc ^ swz(row)) * 8;
    return *(const bf16x8*)(st + row * PITCH + pc * 8);
  }
  // write everything put() since the last flush: dst(row, col) -> destination of 8 columns,
  // or nullptr to drop them.  STREAM: the data is not read again soon (weight gradients), so
  // the stores are marked non-temporal and leave the kernel's inputs in the caches.
  template <bool STREAM = false, class Dst>
  __device__ __forceinline__ void flush(Dst dst) const {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col;
      const bf16x8 v = get(p, row, col);
      bf16* d = dst(row, col);
      if (d != nullptr) {
        if (STREAM) __builtin_nontemporal_store(v, (bf16x8*)d);
        else *(bf16x8*)d = v;
      }
    }
  }
};

}  // namespace momoe
