// Measurement tool, not part of the library: the rate at which this machine sustains bf16
// MFMAs when nothing else happens (operands held in registers, every CU busy, 8 waves per
// CU).  It prints the achieved TFLOP/s and the shader clock during the run (clock64() ticks per
// 100 MHz wall_clock64() tick) for three kinds of operand data: Gaussian values as the layer
// sees them (activations N(0,1) times weights N(0,0.02)), values with random sign and mantissa
// but one exponent, and zeros.  The rate follows how many operand bits toggle: the MFMA pipe is
// power-limited.  The rooflines of the GEMM kernels are read against these figures as well as
// against the published peak.
//
//   python momoe-impl_amd/build.py && momoe-impl_amd/probes/mfma_rate
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kOperandWords = 4096;

// WIDE: v_mfma_f32_32x32x16_bf16 on a 64x128 wave tile (the shape the GEMM kernels use);
// otherwise v_mfma_f32_16x16x32_bf16 on the same tile.  Both do 16 x 32768 flops per iteration.
template <bool WIDE>
__global__ __launch_bounds__(512, 2) void mfma_loop(const uint4* src, const uint4* src_b,
                                                     float* sink, unsigned long long* clocks,
                                                     int iters) {
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  bf16x8 a[8], b[4];
  for (int i = 0; i < 8; ++i)
    a[i] = __builtin_bit_cast(bf16x8, src[(threadIdx.x * 8 + i) % kOperandWords]);
  for (int i = 0; i < 4; ++i)
    b[i] = __builtin_bit_cast(bf16x8, src_b[(threadIdx.x * 4 + i + 977) % kOperandWords]);
  float keep = 0;
  if (WIDE) {
    f32x16 acc[2][4] = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[2 * kk + j], a[4 * kk + i],
                                                                acc[j][i], 0, 0, 0);
    }
    for (int j = 0; j < 2; ++j)
      for (int i = 0; i < 4; ++i)
        for (int r = 0; r < 16; ++r) keep += acc[j][i][r];
  } else {
    f32x4 acc[4][8] = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j], a[i], acc[j][i], 0, 0, 0);
    }
    for (int j = 0; j < 4; ++j)
      for (int i = 0; i < 8; ++i)
        for (int r = 0; r < 4; ++r) keep += acc[j][i][r];
  }
  if (keep == 12345.f) sink[threadIdx.x] = keep;  // keeps the loop alive, never true in practice
  if (blockIdx.x == 17 && threadIdx.x == 0) {
    clocks[0] = clock64() - c0;
    clocks[1] = wall_clock64() - w0;
  }
}

#define CHECK(call)                                                                  \
  do {                                                                               \
    hipError_t e_ = (call);                                                          \
    if (e_ != hipSuccess) {                                                          \
      fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));              \
      return 1;                                                                      \
    }                                                                                \
  } while (0)

template <bool WIDE>
int run(const char* name, int cus, const uint4* src, const uint4* src_b, float* sink,
        unsigned long long* clocks) {
  const int iters = 20000, reps = 3;
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  mfma_loop<WIDE><<<cus, 512>>>(src, src_b, sink, clocks, iters);
  CHECK(hipEventRecord(e0));
  for (int r = 0; r < reps; ++r) mfma_loop<WIDE><<<cus, 512>>>(src, src_b, sink, clocks, iters);
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, e0, e1));
  ms /= reps;
  unsigned long long hc[2];
  CHECK(hipMemcpy(hc, clocks, sizeof(hc), hipMemcpyDeviceToHost));
  const double flops = (double)cus * 8 * iters * 16 * 32768.0;
  printf("%-46s %8.3f ms %7.0f TFLOP/s  shader clock %5.0f MHz\n", name, ms, flops / ms / 1e9,
         (double)hc[0] / (double)hc[1] * 100.0);
  return 0;
}

int main() {
  int cus = 0;
  CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
  // three data sets of kOperandWords 16-byte words each, for the two operands
  const size_t n = (size_t)kOperandWords * 4;
  std::vector<uint32_t> gauss_a(n), gauss_b(n), mant(n), zero(n, 0);
  uint32_t st = 99;
  auto uniform01 = [&] {
    st = st * 1664525u + 1013904223u;
    return ((st >> 8) + 0.5) / 16777216.0;
  };
  auto bf16_bits = [](float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;  // round to nearest even
  };
  auto normal = [&](double sigma) {
    return (float)(sigma * sqrt(-2.0 * log(uniform01())) * cos(6.283185307179586 * uniform01()));
  };
  for (size_t i = 0; i < n; ++i) {
    gauss_a[i] = bf16_bits(normal(1.0)) | (bf16_bits(normal(1.0)) << 16);
    gauss_b[i] = bf16_bits(normal(0.02)) | (bf16_bits(normal(0.02)) << 16);
    st = st * 1664525u + 1013904223u;  // random sign and mantissa, magnitude 1..2
    mant[i] = (0x3F80 | ((st >> 8) & 0x807F)) | ((0x3F80 | ((st >> 20) & 0x807F)) << 16);
  }
  const std::vector<uint32_t>* host[4] = {&gauss_a, &gauss_b, &mant, &zero};
  uint4* dev[4];
  for (int i = 0; i < 4; ++i) {
    CHECK(hipMalloc(&dev[i], n * 4));
    CHECK(hipMemcpy(dev[i], host[i]->data(), n * 4, hipMemcpyHostToDevice));
  }
  float* sink;
  unsigned long long* clocks;
  CHECK(hipMalloc(&sink, 4096));
  CHECK(hipMalloc(&clocks, 16));
  printf("%d CUs, 8 waves per CU, operands in registers\n", cus);
  for (int r = 0; r < 2; ++r) {
    if (run<true>("v_mfma_f32_32x32x16_bf16, N(0,1) x N(0,0.02)", cus, dev[0], dev[1], sink, clocks)) return 1;
    if (run<true>("v_mfma_f32_32x32x16_bf16, one exponent", cus, dev[2], dev[2], sink, clocks)) return 1;
    if (run<true>("v_mfma_f32_32x32x16_bf16, zeros", cus, dev[3], dev[3], sink, clocks)) return 1;
    if (run<false>("v_mfma_f32_16x16x32_bf16, N(0,1) x N(0,0.02)", cus, dev[0], dev[1], sink, clocks)) return 1;
    if (run<false>("v_mfma_f32_16x16x32_bf16, one exponent", cus, dev[2], dev[2], sink, clocks)) return 1;
    if (run<false>("v_mfma_f32_16x16x32_bf16, zeros", cus, dev[3], dev[3], sink, clocks)) return 1;
  }
  return 0;
}
