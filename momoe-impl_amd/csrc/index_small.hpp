// The routing index of a decode-sized call, built by one workgroup: at most 256 tokens (one
// token panel) and 256 experts.  Shared by the one-launch index kernel and by the x.Wl1 kernel for
// small calls, whose workgroups each build the index for themselves instead of waiting for a
// separate launch.
//
// Thread t < 256 is token t and reads its whole mask column up front (all loads in flight at
// once: one memory latency), as 16 bits per group of 16 experts; one ballot per expert gives the
// lane masks of its tokens, a scan over the experts gives the prefix sums and the tile table, and
// every token then places its own K pairs from its bits and those masks.
#pragma once
#include "common.hpp"

namespace momoe {

constexpr int kPanelTokens = 256;
constexpr int kPanelExperts = 16;
constexpr int kSmallMaxGroups = 16;
constexpr int kSmallMaxExperts = kSmallMaxGroups * kPanelExperts;
static_assert(kPanelTokens <= MOMOE_RECOMPUTE_TILE_ROWS, "one tile per expert in the one-workgroup build");

// The 16 mask entries of token m in expert group g, as a bit set.  Loads are unconditional (row
// and column clamped into the matrix, the result masked afterwards): a load under a branch is
// waited for before the next one is issued, which made this function one memory latency PER
// ENTRY instead of one per group.
__device__ __forceinline__ uint32_t load_panel_bits(const int32_t* __restrict__ mask, int64_t sn,
                                                    int64_t sm, int M, int N, int g, int m) {
  const int32_t* col = mask + (int64_t)min(m, M - 1) * sm;
  int32_t v[kPanelExperts];
#pragma unroll
  for (int e = 0; e < kPanelExperts; ++e)
    v[e] = col[(int64_t)min(g * kPanelExperts + e, N - 1) * sn];
  uint32_t bits = 0;
#pragma unroll
  for (int e = 0; e < kPanelExperts; ++e)
    bits |= (v[e] != 0 && g * kPanelExperts + e < N ? 1u : 0u) << e;
  return m < M ? bits : 0u;
}

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int o = __shfl_up(v, d);
    if (lane >= d) v += o;
  }
  return v;
}

// What the build keeps in LDS.  `cum` (exclusive prefix sums of the experts' rows, cum[n] = all
// pairs), `act` (the experts that hold a token, ascending) and `nact` stay valid after the build.
template <int NGROUPS>
struct SmallIndexLds {
  static constexpr int kExperts = NGROUPS * kPanelExperts;
  uint64_t ball[kExperts][4];  // tokens of expert i in wave w, as a lane mask
  int32_t cum[kExperts + 1];
  int32_t act[kExperts];
  int32_t wave_sums[4][3];     // per wave of experts: rows, row tiles, experts with a token
  int32_t nact, total;
};

// Global outputs of the build (momoe_index_build's); written when `write` is set.
struct SmallIndexOut {
  int64_t* sizes;
  int32_t* cumsums;
  int32_t* idx;
  int32_t* which;
  int32_t* inv;
  int32_t* table;
  int32_t* violations;
  bool write;
};

// Every thread of the workgroup calls this (it holds barriers); threads 0..255 are the tokens,
// further threads only keep the barriers.  lds_idx: if not null, LDS array of M*K ints that
// receives the token of every sorted row (the caller guarantees M*K entries).  tile_rows: 0 = 256.
// With at most 256 tokens no expert holds more than 256 rows: taller tiles would save nothing.
// On return (after a barrier) L.cum / L.act / L.nact / L.total and lds_idx are complete; with more
// pairs than M*K (a routing the layer refuses) L.nact is 0.
template <int NGROUPS>
__device__ __forceinline__ void small_index_build(const int32_t* __restrict__ mask, int64_t sn, int64_t sm,
                                                  int M, int N, int K, int tile_rows_arg,
                                                  SmallIndexLds<NGROUPS>& L, int32_t* lds_idx,
                                                  const SmallIndexOut& out) {
  const int tile_rows = tile_rows_arg > 0 ? tile_rows_arg : MOMOE_RECOMPUTE_TILE_ROWS;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const bool token_thread = t < kPanelTokens;  // wave-uniform
  const int64_t msum = (int64_t)M * K;
  uint32_t bits[NGROUPS];
  if (token_thread) {
#pragma unroll
    for (int g = 0; g < NGROUPS; ++g) bits[g] = load_panel_bits(mask, sn, sm, M, N, g, t);
#pragma unroll
    for (int g = 0; g < NGROUPS; ++g)
#pragma unroll
      for (int e = 0; e < kPanelExperts; ++e) {
        const uint64_t b = __ballot((bits[g] >> e) & 1u);
        if (lane == 0) L.ball[g * kPanelExperts + e][wave] = b;
      }
  }
  __syncthreads();
  // exclusive scan over the experts of (rows, row tiles, experts with a token): one expert per thread
  int v = 0, nt = 0, nz = 0, irows = 0, itiles = 0, inz = 0;
  if (token_thread) {
    v = t < N ? __popcll(L.ball[t][0]) + __popcll(L.ball[t][1]) + __popcll(L.ball[t][2]) + __popcll(L.ball[t][3]) : 0;
    nt = (v + tile_rows - 1) / tile_rows;
    nz = v > 0 ? 1 : 0;
    irows = wave_inclusive_scan(v, lane);
    itiles = wave_inclusive_scan(nt, lane);
    inz = wave_inclusive_scan(nz, lane);
    if (lane == 63) {
      L.wave_sums[wave][0] = irows;
      L.wave_sums[wave][1] = itiles;
      L.wave_sums[wave][2] = inz;
    }
  }
  __syncthreads();
  const int total = L.wave_sums[0][0] + L.wave_sums[1][0] + L.wave_sums[2][0] + L.wave_sums[3][0];
  const int total_tiles = L.wave_sums[0][1] + L.wave_sums[1][1] + L.wave_sums[2][1] + L.wave_sums[3][1];
  const int total_nz = L.wave_sums[0][2] + L.wave_sums[1][2] + L.wave_sums[2][2] + L.wave_sums[3][2];
  const bool overflow = (int64_t)total > msum;
  if (token_thread) {
    int brow = irows - v, btile = itiles - nt, bnz = inz - nz;
    for (int w = 0; w < wave; ++w) {
      brow += L.wave_sums[w][0];
      btile += L.wave_sums[w][1];
      bnz += L.wave_sums[w][2];
    }
    if (t < SmallIndexLds<NGROUPS>::kExperts) L.cum[t] = brow;
    if (t < N && nz && !overflow) L.act[bnz] = t;
    if (t == 0) {
      L.cum[SmallIndexLds<NGROUPS>::kExperts] = total;
      L.nact = overflow ? 0 : total_nz;
      L.total = total;
    }
    if (out.write) {
      if (t < N) {
        out.cumsums[t] = brow;
        out.sizes[t] = (int64_t)v;
        if (!overflow)
          for (int k = 0; k < nt; ++k) {
            int32_t* e = out.table + kTileHeader + 4 * (btile + k);
            e[0] = t;
            e[1] = btile;
            e[2] = brow;
            e[3] = v;
          }
      }
      if (t == 0) {
        out.cumsums[N] = total;
        if (overflow) atomicAdd(out.violations, 1);
        out.table[0] = overflow ? 0 : total_tiles;
        out.table[1] = tile_rows;
        out.table[2] = 0;
        out.table[3] = 0;
      }
      // sorted rows past the last pair (a routing with fewer than M*K pairs): token 0, slot 0
      for (int64_t r = (int64_t)total + t; r < msum; r += kPanelTokens) {
        out.idx[r] = 0;
        out.which[r] = 0;
      }
    }
    if (lds_idx != nullptr)
      for (int64_t r = (int64_t)total + t; r < msum; r += kPanelTokens) lds_idx[r] = 0;
  }
  __syncthreads();
  if (token_thread) {
    // every token walks its own pairs (K of them, not N candidates), lowest expert first
    const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    int k = 0;
#pragma unroll
    for (int g = 0; g < NGROUPS; ++g) {
      uint32_t rest = bits[g];
      while (rest != 0) {
        const int i = g * kPanelExperts + __ffs(rest) - 1;
        rest &= rest - 1;
        int before = __popcll(L.ball[i][wave] & below);
        for (int w = 0; w < wave; ++w) before += __popcll(L.ball[i][w]);
        const int64_t row = (int64_t)L.cum[i] + before;
        if (row < msum) {
          if (lds_idx != nullptr) lds_idx[row] = t;
          if (out.write) {
            out.idx[row] = t;
            out.which[row] = k;
          }
        }
        if (out.write && k < K) out.inv[(int64_t)t * K + k] = row < msum && !overflow ? (int32_t)row : -1;
        ++k;
      }
    }
    if (out.write && t < M && k != K) {
      atomicAdd(out.violations, 1);
      for (int kk = k; kk < K; ++kk) out.inv[(int64_t)t * K + kk] = -1;
    }
  }
  __syncthreads();
}

}  // namespace momoe
