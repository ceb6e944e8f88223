// Top-k + softmax router with selection bias and shared experts: the elementwise
// part of the forward (everything after the gate GEMM) and the backward through
// renormalisation and softmax.  One wavefront per token; lane j holds columns
// j, j+64, ...  HBM-bound: a few passes over [M, N] fp32.
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

__global__ __launch_bounds__(256) void router_fwd_kernel(RouterFwdArgs p) {
  const int lane = threadIdx.x & 63;
  const int m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= p.M) return;
  const int N = p.N, Ng = p.N - p.Ks, Kg = p.K - p.Ks;
  const int ncol = (N + 63) >> 6;
  float v[kMaxCols], pr[kMaxCols], score[kMaxCols];
  bool sel[kMaxCols];
  float mg = -INFINITY, ms = -INFINITY;
#pragma unroll
  for (int c = 0; c < kMaxCols; ++c) {
    const int j = lane + 64 * c;
    v[c] = -INFINITY;
    if (c < ncol && j < N) {
      v[c] = p.logits_f32 ? ((const float*)p.logits)[(int64_t)m * N + j]
                          : (float)((const bf16*)p.logits)[(int64_t)m * N + j];
      if (j < Ng) mg = fmaxf(mg, v[c]); else ms = fmaxf(ms, v[c]);
    }
  }
  mg = wave_max(mg);
  ms = wave_max(ms);
  float sg = 0.0f, ss = 0.0f;
#pragma unroll
  for (int c = 0; c < kMaxCols; ++c) {
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
  for (int c = 0; c < kMaxCols; ++c) {
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
    for (int c = 0; c < kMaxCols; ++c) {
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
    for (int c = 0; c < kMaxCols; ++c)
      if (lane + 64 * c == bj) sel[c] = true;
  }
  float ngsum = 0.0f, kssum = 0.0f;
#pragma unroll
  for (int c = 0; c < kMaxCols; ++c) {
    const int j = lane + 64 * c;
    if (c < ncol && j < N) {
      if (j < Ng) ngsum += sel[c] ? pr[c] : 0.0f; else kssum += pr[c];
    }
  }
  ngsum = wave_sum(ngsum);
  kssum = wave_sum(kssum);
#pragma unroll
  for (int c = 0; c < kMaxCols; ++c) {
    const int j = lane + 64 * c;
    if (c < ncol && j < N) {
      const bool routed = j < Ng;
      const bool on = routed ? sel[c] : true;
      const float pv = on ? pr[c] : 0.0f;
      p.psel[(int64_t)m * N + j] = pv;
      p.s[(int64_t)m * N + j] = routed ? pv / ngsum : pv / kssum;
      p.mask[(int64_t)j * p.M + m] = on ? 1 : 0;
    }
  }
  if (lane == 0) {
    p.ng[m] = ngsum;
    p.ks[m] = kssum;
  }
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

__global__ __launch_bounds__(256) void router_bwd_kernel(RouterBwdArgs p) {
  const int lane = threadIdx.x & 63;
  const int m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= p.M) return;
  const int N = p.N, Ng = p.N - p.Ks;
  const int ncol = (N + 63) >> 6;
  float g[kMaxCols], pv[kMaxCols];
  float dotg = 0.0f, dots = 0.0f;
#pragma unroll
  for (int c = 0; c < kMaxCols; ++c) {
    const int j = lane + 64 * c;
    g[c] = 0.0f;
    pv[c] = 0.0f;
    if (c < ncol && j < N) {
      g[c] = p.gs[(int64_t)j * p.gsn + (int64_t)m * p.gsm];
      pv[c] = p.psel[(int64_t)m * N + j];
      const float sv = p.s[(int64_t)m * N + j];
      if (j < Ng) dotg += p.mask[(int64_t)j * p.M + m] != 0 ? g[c] * sv : 0.0f;
      else dots += g[c] * sv;
    }
  }
  dotg = wave_sum(dotg);
  dots = wave_sum(dots);
  const float ing = 1.0f / p.ng[m];
  const float iks = p.Ks > 0 ? 1.0f / p.ks[m] : 0.0f;
  float o[kMaxCols];
  float inner_g = 0.0f, inner_s = 0.0f;
#pragma unroll
  for (int c = 0; c < kMaxCols; ++c) {
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
  for (int c = 0; c < kMaxCols; ++c) {
    const int j = lane + 64 * c;
    if (c < ncol && j < N)
      p.out[(int64_t)m * N + j] = (bf16)(pv[c] * (o[c] - (j < Ng ? inner_g : inner_s)));
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
  router_fwd_kernel<<<(unsigned)cdiv64(M, 4), 256, 0, (hipStream_t)stream>>>(a);
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
  router_bwd_kernel<<<(unsigned)cdiv64(M, 4), 256, 0, (hipStream_t)stream>>>(a);
  return launch_status();
}
