// Top-k + softmax router with selection bias and shared experts: the elementwise
// part of the forward (everything after the gate GEMM) and the backward through
// renormalisation and softmax.  One wavefront per token (lane j holds columns
// j, j+64, ...), a workgroup per block of consecutive tokens so that the [N, M]
// tensors (mask, dL/ds) are touched in whole lines.  HBM-bound: a few passes over
// [M, N] fp32.
#include "common.hpp"

namespace momoe {
namespace {

constexpr int kMaxCols = 8;  // columns per lane -> N <= 512

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v = fmaxf(v, __shfl_xor(v, d));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
  return v;
}

struct RouterFwdArgs {
  const void* logits;
  int logits_f32;
  const float* bias;
  int M, N, K, Ks;
  int32_t* mask;
  float* s;
  float* psel;
  float* ng;
  float* ks;
};

// A workgroup of 16 wavefronts handles kTok = 32 consecutive tokens, two per wavefront.  The
// mask is [N, M] (token fastest) while everything else is per token: the 0/1 flags of the 32
// tokens go through LDS and leave as rows of 32 x 4 bytes, whole 128-byte lines (written per
// token they would be N scattered 4-byte stores each).
constexpr int kTok = 32;
constexpr int kRouterThreads = 1024;

// NC = columns held per lane (1, 2, 4 or 8): N <= 64 * NC
template <int NC>
__global__ __launch_bounds__(kRouterThreads) void router_fwd_kernel(RouterFwdArgs p) {
  __shared__ uint8_t flags[64 * NC][kTok];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int N = p.N, Ng = p.N - p.Ks, Kg = p.K - p.Ks;
  const int ncol = (N + 63) >> 6;
  const int m0 = blockIdx.x * kTok;
  for (int tt = wave; tt < kTok; tt += kRouterThreads / 64) {
    const int m = m0 + tt;
    if (m >= p.M) break;  // wave-uniform
    float v[NC], pr[NC], score[NC];
    bool sel[NC];
    float mg = -INFINITY, ms = -INFINITY;
    // unconditional loads (column clamped, result masked): loads under a branch would be
    // waited for one by one
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int jc = min(lane + 64 * min(c, ncol - 1), N - 1);
      v[c] = p.logits_f32 ? ((const float*)p.logits)[(int64_t)m * N + jc]
                          : (float)((const bf16*)p.logits)[(int64_t)m * N + jc];
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int j = lane + 64 * c;
      if (c < ncol && j < N) {
        if (j < Ng) mg = fmaxf(mg, v[c]); else ms = fmaxf(ms, v[c]);
      } else {
        v[c] = -INFINITY;
      }
    }
    mg = wave_max(mg);
    ms = wave_max(ms);
    float sg = 0.0f, ss = 0.0f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int j = lane + 64 * c;
      pr[c] = 0.0f;
      if (c < ncol && j < N) {
        pr[c] = expf(v[c] - (j < Ng ? mg : ms));
        if (j < Ng) sg += pr[c]; else ss += pr[c];
      }
    }
    sg = wave_sum(sg);
    ss = wave_sum(ss);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int j = lane + 64 * c;
      sel[c] = false;
      score[c] = -INFINITY;
      if (c < ncol && j < N) {
        pr[c] = pr[c] / (j < Ng ? sg : ss);
        if (j < Ng) score[c] = pr[c] + p.bias[j];
      }
    }
    // top-Kg of score over the routed columns; ties go to the lower column
    for (int round = 0; round < Kg; ++round) {
      float bv = -INFINITY;
      int bj = 0x7fffffff;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int j = lane + 64 * c;
        if (c < ncol && j < Ng && !sel[c] && (score[c] > bv || (score[c] == bv && j < bj))) {
          bv = score[c];
          bj = j;
        }
      }
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) {
        const float ov = __shfl_xor(bv, d);
        const int oj = __shfl_xor(bj, d);
        if (ov > bv || (ov == bv && oj < bj)) {
          bv = ov;
          bj = oj;
        }
      }
#pragma unroll
      for (int c = 0; c < NC; ++c)
        if (lane + 64 * c == bj) sel[c] = true;
    }
    float ngsum = 0.0f, kssum = 0.0f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int j = lane + 64 * c;
      if (c < ncol && j < N) {
        if (j < Ng) ngsum += sel[c] ? pr[c] : 0.0f; else kssum += pr[c];
      }
    }
    ngsum = wave_sum(ngsum);
    kssum = wave_sum(kssum);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int j = lane + 64 * c;
      if (c < ncol && j < N) {
        const bool routed = j < Ng;
        const bool on = routed ? sel[c] : true;
        const float pv = on ? pr[c] : 0.0f;
        p.psel[(int64_t)m * N + j] = pv;
        p.s[(int64_t)m * N + j] = routed ? pv / ngsum : pv / kssum;
        flags[j][tt] = on ? 1 : 0;
      }
    }
    if (lane == 0) {
      p.ng[m] = ngsum;
      p.ks[m] = kssum;
    }
  }
  __syncthreads();
  // mask rows: 32 tokens x 4 bytes per expert
  const int tt = threadIdx.x & (kTok - 1);
  if (m0 + tt < p.M)
    for (int j = threadIdx.x / kTok; j < N; j += kRouterThreads / kTok)
      p.mask[(int64_t)j * p.M + m0 + tt] = flags[j][tt];
}

struct RouterBwdArgs {
  const float* gs;
  int64_t gsn, gsm;
  const float* psel;
  const float* s;
  const float* ng;
  const float* ks;
  const int32_t* mask;
  int M, N, Ks;
  bf16* out;
};

// TB consecutive tokens per workgroup of 16 wavefronts.  dL/ds and the mask are [N, M]: a token's
// column is N scattered 4-byte reads, so the TB columns are first copied to LDS with loads that
// run along whichever index is contiguous in memory, and the per-token pass reads them there.
template <int TB, int NC>
__global__ __launch_bounds__(kRouterThreads) void router_bwd_kernel(RouterBwdArgs p) {
  constexpr int kTileFloats = 512 * 17;  // N <= 512 with TB = 16 (8704), N <= 256 with TB = 32 (8448)
  static_assert(TB == 32 || TB == 16, "tile sizes the LDS arrays are cut for");
  __shared__ float gs_t[kTileFloats];       // [N][TB + 1]
  __shared__ uint8_t mk_t[256 * 32];        // [N][TB]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int N = p.N, Ng = p.N - p.Ks;
  const int ncol = (N + 63) >> 6;
  const int m0 = blockIdx.x * TB;
  const int ntok = min(TB, p.M - m0);
  if (p.gsm == 1) {  // tokens contiguous: [N, M] as the experts' backward writes it
    for (int q = threadIdx.x; q < N * TB; q += kRouterThreads) {
      const int j = q / TB, tt = q % TB;
      if (tt < ntok) gs_t[j * (TB + 1) + tt] = p.gs[(int64_t)j * p.gsn + m0 + tt];
    }
  } else {           // any other strides: run along the experts
    for (int q = threadIdx.x; q < N * TB; q += kRouterThreads) {
      const int tt = q / N, j = q % N;
      if (tt < ntok) gs_t[j * (TB + 1) + tt] = p.gs[(int64_t)j * p.gsn + (int64_t)(m0 + tt) * p.gsm];
    }
  }
  for (int q = threadIdx.x; q < N * TB; q += kRouterThreads) {
    const int j = q / TB, tt = q % TB;
    if (tt < ntok) mk_t[j * TB + tt] = p.mask[(int64_t)j * p.M + m0 + tt] != 0;
  }
  __syncthreads();
  for (int tt = wave; tt < ntok; tt += kRouterThreads / 64) {
    const int m = m0 + tt;
    float g[NC], pv[NC], sv[NC];
    float dotg = 0.0f, dots = 0.0f;
    // unconditional loads (column clamped, results masked), all issued before any is used
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int jc = min(lane + 64 * min(c, ncol - 1), N - 1);
      pv[c] = p.psel[(int64_t)m * N + jc];
      sv[c] = p.s[(int64_t)m * N + jc];
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int j = lane + 64 * c;
      g[c] = 0.0f;
      if (c < ncol && j < N) {
        g[c] = gs_t[j * (TB + 1) + tt];
        if (j < Ng) dotg += mk_t[j * TB + tt] ? g[c] * sv[c] : 0.0f;
        else dots += g[c] * sv[c];
      } else {
        pv[c] = 0.0f;
      }
    }
    dotg = wave_sum(dotg);
    dots = wave_sum(dots);
    const float ing = 1.0f / p.ng[m];
    const float iks = p.Ks > 0 ? 1.0f / p.ks[m] : 0.0f;
    float o[NC];
    float inner_g = 0.0f, inner_s = 0.0f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int j = lane + 64 * c;
      o[c] = 0.0f;
      if (c < ncol && j < N) {
        if (j < Ng) {
          o[c] = (g[c] - dotg) * ing;
          inner_g += o[c] * pv[c];
        } else {
          o[c] = (g[c] - dots) * iks;
          inner_s += o[c] * pv[c];
        }
      }
    }
    inner_g = wave_sum(inner_g);
    inner_s = wave_sum(inner_s);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int j = lane + 64 * c;
      if (c < ncol && j < N)
        p.out[(int64_t)m * N + j] = (bf16)(pv[c] * (o[c] - (j < Ng ? inner_g : inner_s)));
    }
  }
}

}  // namespace
}  // namespace momoe

using namespace momoe;

extern "C" int momoe_router_fwd(const void* logits_MN, int logits_f32, const float* biases_N,
                                int64_t M, int64_t N, int64_t K, int64_t Ks, int32_t* mask_NM,
                                float* s_MN, float* p_sel_MN, float* Ng_M, float* Ks_M,
                                void* stream) {
  if (!logits_MN || !biases_N || !mask_NM || !s_MN || !p_sel_MN || !Ng_M || !Ks_M)
    return MOMOE_ERR_BAD_ARG;
  if (M <= 0 || N <= 0 || Ks < 0 || K < Ks || Ks > N || K - Ks > N - Ks) return MOMOE_ERR_BAD_ARG;
  if (N > 64 * kMaxCols || M >= (1ll << 31) - 4) return MOMOE_ERR_UNSUPPORTED;
  RouterFwdArgs a{logits_MN, logits_f32, biases_N, (int)M, (int)N, (int)K, (int)Ks,
                  mask_NM, s_MN, p_sel_MN, Ng_M, Ks_M};
  const unsigned grid = (unsigned)cdiv64(M, kTok);
  hipStream_t st = (hipStream_t)stream;
  if (N <= 64) router_fwd_kernel<1><<<grid, kRouterThreads, 0, st>>>(a);
  else if (N <= 128) router_fwd_kernel<2><<<grid, kRouterThreads, 0, st>>>(a);
  else if (N <= 256) router_fwd_kernel<4><<<grid, kRouterThreads, 0, st>>>(a);
  else router_fwd_kernel<8><<<grid, kRouterThreads, 0, st>>>(a);
  return launch_status();
}

extern "C" int momoe_router_bwd(const float* Gs_NM, int64_t gs_stride_n, int64_t gs_stride_m,
                                const float* p_sel_MN, const float* s_MN, const float* Ng_M,
                                const float* Ks_M, const int32_t* mask_NM, int64_t M, int64_t N,
                                int64_t Ks, void* Glogits_MN, void* stream) {
  if (!Gs_NM || !p_sel_MN || !s_MN || !Ng_M || !Ks_M || !mask_NM || !Glogits_MN)
    return MOMOE_ERR_BAD_ARG;
  if (M <= 0 || N <= 0 || Ks < 0 || Ks > N) return MOMOE_ERR_BAD_ARG;
  if (N > 64 * kMaxCols || M >= (1ll << 31) - 4) return MOMOE_ERR_UNSUPPORTED;
  RouterBwdArgs a{Gs_NM, gs_stride_n, gs_stride_m, p_sel_MN, s_MN, Ng_M, Ks_M, mask_NM,
                  (int)M, (int)N, (int)Ks, (bf16*)Glogits_MN};
  hipStream_t st = (hipStream_t)stream;
  const unsigned grid32 = (unsigned)cdiv64(M, 32);
  if (N <= 64) router_bwd_kernel<32, 1><<<grid32, kRouterThreads, 0, st>>>(a);
  else if (N <= 128) router_bwd_kernel<32, 2><<<grid32, kRouterThreads, 0, st>>>(a);
  else if (N <= 256) router_bwd_kernel<32, 4><<<grid32, kRouterThreads, 0, st>>>(a);
  else router_bwd_kernel<16, 8><<<(unsigned)cdiv64(M, 16), kRouterThreads, 0, st>>>(a);
  return launch_status();
}
