// Version and status strings of the C ABI.
#include <atomic>

#include "gemm_tile.hpp"

namespace momoe {
namespace {
std::atomic<unsigned long long*> g_clock_trace{nullptr};
}
unsigned long long* clock_trace_buffer() { return g_clock_trace.load(std::memory_order_relaxed); }
}  // namespace momoe

extern "C" int momoe_abi_version(void) { return 3; }

extern "C" const char* momoe_status_string(int status) {
  switch (status) {
    case MOMOE_OK: return "ok";
    case MOMOE_ERR_BAD_ARG: return "bad argument (null/misaligned pointer or non-positive size)";
    case MOMOE_ERR_UNSUPPORTED: return "unsupported shape";
    case MOMOE_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}

extern "C" int momoe_set_clock_trace(unsigned long long* ticks2) {
  momoe::g_clock_trace.store(ticks2, std::memory_order_relaxed);
  return MOMOE_OK;
}

namespace momoe {
namespace {
// Nothing but the GEMMs' MFMA on operands held in registers, the accumulator tile of one wave of
// the grouped GEMMs (2 x 4 fragments), 8 waves per CU: the rate the matrix pipe sustains on the
// given operand data when nothing else draws power or issue slots.
__global__ __launch_bounds__(kThreads, 2) void mfma_rate_kernel(const u32x4* __restrict__ operands,
                                                                float* __restrict__ sink, int iters,
                                                                unsigned long long* __restrict__ ticks2) {
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  bf16x8 a[8], b[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = __builtin_bit_cast(bf16x8, operands[(threadIdx.x * 8 + i) % 2048]);
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = __builtin_bit_cast(bf16x8, operands[2048 + (threadIdx.x * 4 + i + 977) % 2048]);
  f32x16 acc[2][4];
  zero_acc<4, 2>(acc);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[j][i] = mfma32(b[2 * kk + j], a[4 * kk + i], acc[j][i]);
  }
  float keep = 0.0f;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) keep += acc[j][i][r];
  if (keep == 12345.0f) sink[threadIdx.x] = keep;  // never true on the data this is used with
  if (ticks2 != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
    ticks2[0] = clock64() - c0;
    ticks2[1] = wall_clock64() - w0;
  }
}
// Nothing but the weight stream of the grouped GEMMs: global -> LDS transfers of [32 k-rows] x
// [256 columns] stages of a row-major matrix, a ring of four stages per workgroup, one workgroup
// per CU walking (matrix, column block) tiles; nothing reads the data.
__global__ __launch_bounds__(kThreads) void hbm_stream_kernel(const bf16* __restrict__ w, int64_t blocks,
                                                              int krows, int ncol) {
  constexpr int S = 4;
  TDma B;
  const uint32_t lds = lds_address(dyn_lds());
  const int nb = ncol / TLayout::COLS, ktiles = krows / kBK;
  for (int64_t t = blockIdx.x; t < blocks * nb; t += gridDim.x) {
    const int64_t e = t / nb;
    const int tn = (int)(t % nb);
    B.init(w + e * krows * ncol, [&](int c) { return tn * TLayout::COLS + c; }, ncol);
    for (int s = 0; s < S - 1 && s < ktiles; ++s) B.issue(s, lds + s * (TLayout::LDS_ELEMS * 2));
    for (int kt = 0; kt < ktiles; ++kt) {
      if (kt + S - 1 < ktiles) {
        B.issue(kt + S - 1, lds + ((kt + S - 1) % S) * (TLayout::LDS_ELEMS * 2));
        wait_vmcnt<(S - 1) * TDma::NCH>();
      } else {
        wait_vmcnt<0>();
      }
      __builtin_amdgcn_s_barrier();
    }
  }
}
}  // namespace
}  // namespace momoe

extern "C" int64_t momoe_hbm_stream_probe(const void* matrix, int64_t blocks, int64_t krows,
                                          int64_t ncol, void* stream) {
  if (!matrix || blocks <= 0 || krows <= 0 || ncol <= 0 || ((uintptr_t)matrix & 15)) return -1;
  if (krows % momoe::kBK != 0 || ncol % momoe::TLayout::COLS != 0 || krows * ncol * 2 >= (1ll << 32))
    return -1;
  momoe::hbm_stream_kernel<<<momoe::persistent_grid(), momoe::kThreads, 4 * momoe::TLayout::LDS_ELEMS * 2,
                             (hipStream_t)stream>>>((const momoe::bf16*)matrix, blocks, (int)krows, (int)ncol);
  if (hipGetLastError() != hipSuccess) return -1;
  return blocks * krows * ncol * 2;
}

extern "C" int64_t momoe_mfma_rate_probe(const void* operands_64KiB, float* sink_512, int iters,
                                         unsigned long long* ticks2, void* stream) {
  if (!operands_64KiB || !sink_512 || iters <= 0 || ((uintptr_t)operands_64KiB & 15)) return -1;
  const int grid = momoe::persistent_grid();
  momoe::mfma_rate_kernel<<<grid, momoe::kThreads, 0, (hipStream_t)stream>>>(
      (const momoe::u32x4*)operands_64KiB, sink_512, iters, ticks2);
  if (hipGetLastError() != hipSuccess) return -1;
  // flops of the launch: workgroups x 8 waves x iterations x 16 MFMAs of 2 * 32 * 32 * 16
  return (int64_t)grid * momoe::kWaves * iters * 16 * 32768;
}
