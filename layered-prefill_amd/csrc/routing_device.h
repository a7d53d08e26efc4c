// Device side of the router shared by the kernels that route rows of E experts with E a power of
// two up to 256 (topk_softmax_pow2_kernel, the gate-fused kernel, the single-workgroup routing +
// alignment kernel): lane geometry, lane exchanges and the softmax + top-k of one row.
#pragma once

#include "common.h"

namespace {

template <int E>
struct Pow2Geom {
  static constexpr int kEpl = (E < 4) ? E : 4;  // floats per vector load
  static constexpr int kVecs = (E / (kEpl * 32)) < 1 ? 1 : (E / (kEpl * 32));
  static constexpr int kVpt = kVecs * kEpl;     // values per lane
  static constexpr int kTpr = E / kVpt;         // lanes per row
  static constexpr int kRowsPerWave = kWave / kTpr;
};

constexpr int kWavesPerBlock = 4;

// Lane exchange for the order-independent reductions (max, argmax): partner at
// distance M inside a row of TPR lanes.  Distances 1 and 2 are exact xor
// butterflies (quad_perm); 4 and 8 use the mirror patterns of DPP, which pair
// every lane with a lane of the other half of its 8- or 16-lane group: the same
// thing once the lanes of each half already agree, which is why these
// reductions run from distance 1 upwards.  DPP moves cost a few clocks; the
// LDS-crossbar shuffle behind __shfl_xor costs ~100 and was most of a round.
template <int M>
__device__ __forceinline__ int lane_exchange(int v) {
  if constexpr (M == 1) return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true);        // quad_perm [1,0,3,2]
  else if constexpr (M == 2) return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
  else if constexpr (M == 4) return __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true);  // row_half_mirror
  else if constexpr (M == 8) return __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, true);  // row_mirror
  else return __shfl_xor(v, M, kWave);
}
template <int M>
__device__ __forceinline__ float lane_exchange(float v) {
  return __builtin_bit_cast(float, lane_exchange<M>(__builtin_bit_cast(int, v)));
}

template <int M, int TPR>
__device__ __forceinline__ void max_level(float& mx) {
  if constexpr (M < TPR) {
    mx = fmaxf(mx, lane_exchange<M>(mx));
    max_level<M * 2, TPR>(mx);
  }
}
template <int M, int TPR>
__device__ __forceinline__ void argmax_level(float& best, int& bidx) {
  if constexpr (M < TPR) {
    const float ov = lane_exchange<M>(best);
    const int oi = lane_exchange<M>(bidx);
    if (ov > best || (ov == best && oi < bidx)) { best = ov; bidx = oi; }
    argmax_level<M * 2, TPR>(best, bidx);
  }
}

// The logits of row `row` as route_row wants them: lane t of the row loads columns
// (i / EPL) * EPL * TPR + t * EPL + i % EPL into v[i], EPL at a time.
template <int E>
__device__ __forceinline__ void load_row(const float* __restrict__ gating, int row, int t,
                                         float (&v)[Pow2Geom<E>::kVpt]) {
  using G = Pow2Geom<E>;
  constexpr int EPL = G::kEpl, VECS = G::kVecs, TPR = G::kTpr;
  const float* src = gating + static_cast<size_t>(row) * E + t * EPL;
#pragma unroll
  for (int j = 0; j < VECS; ++j) {
    if constexpr (EPL == 4) {
      float4 q = *reinterpret_cast<const float4*>(src + j * EPL * TPR);
      v[j * 4 + 0] = q.x; v[j * 4 + 1] = q.y; v[j * 4 + 2] = q.z; v[j * 4 + 3] = q.w;
    } else if constexpr (EPL == 2) {
      float2 q = *reinterpret_cast<const float2*>(src + j * EPL * TPR);
      v[j * 2 + 0] = q.x; v[j * 2 + 1] = q.y;
    } else {
      v[j] = src[j * EPL * TPR];
    }
  }
}

// Softmax and K argmax rounds of one row spread over TPR lanes: lane t of the
// row holds columns (i / EPL) * EPL * TPR + t * EPL + i % EPL in v[i].
template <int E>
__device__ __forceinline__ void route_row(float (&v)[Pow2Geom<E>::kVpt], int t, int row, bool live,
                                          float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
                                          int32_t* __restrict__ tok_exp_idx, int T, int K,
                                          int renormalize) {
  using G = Pow2Geom<E>;
  constexpr int EPL = G::kEpl, VPT = G::kVpt, TPR = G::kTpr;
  float mx = v[0];
#pragma unroll
  for (int i = 1; i < VPT; ++i) mx = fmaxf(mx, v[i]);
  max_level<1, TPR>(mx);

  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    v[i] = moe_expf(v[i] - mx);
    sum += v[i];
  }
#pragma unroll
  for (int m = TPR / 2; m > 0; m /= 2) sum += __shfl_xor(sum, m, kWave);
  const float rinv = 1.f / sum;
#pragma unroll
  for (int i = 0; i < VPT; ++i) v[i] = v[i] * rinv;  // subnormal probabilities are kept, as the reference keeps them

  // Up to kRegK winners stay in registers until the row is done (after the
  // all-reduce every lane of the row knows them): the renormalised weights are
  // then written once, and when the row has at least K lanes, lane k writes
  // winner k, so a row's results leave as three short coalesced stores instead
  // of three single-lane stores per round.
  constexpr int kRegK = 16;
  float wsum = 0.f;
  float bw[kRegK];
  int bi[kRegK];
#pragma unroll
  for (int k = 0; k < kRegK; ++k) { bw[k] = 0.f; bi[k] = 0; }
  auto round = [&](float& best_out, int& bidx_out) {
    float best = v[0];
    int bidx = t * EPL;
#pragma unroll
    for (int i = 1; i < VPT; ++i) {
      const int col = (i / EPL) * (EPL * TPR) + t * EPL + (i % EPL);
      if (v[i] > best) { best = v[i]; bidx = col; }
    }
    argmax_level<1, TPR>(best, bidx);
    wsum += best;
    best_out = best;
    bidx_out = bidx;
    // blank the winner in the lane that holds it
    const int owner = (bidx / EPL) % TPR;
    const int slot = (bidx / (EPL * TPR)) * EPL + (bidx % EPL);
#pragma unroll
    for (int i = 0; i < VPT; ++i)
      if (t == owner && i == slot) v[i] = -10000.f;
  };
  if (K <= kRegK) {
#pragma unroll
    for (int k = 0; k < kRegK; ++k)
      if (k < K) round(bw[k], bi[k]);
    if (K <= TPR) {
      float my_w = 0.f;
      int my_i = 0;
#pragma unroll
      for (int k = 0; k < kRegK; ++k)
        if (t == k) { my_w = bw[k]; my_i = bi[k]; }
      if (live && t < K) {
        const size_t o = static_cast<size_t>(row) * K + t;
        topk_w[o] = renormalize ? my_w / wsum : my_w;
        topk_ids[o] = my_i;
        tok_exp_idx[o] = t * T + row;
      }
    } else if (live && t == 0) {
#pragma unroll
      for (int k = 0; k < kRegK; ++k)
        if (k < K) {
          const size_t o = static_cast<size_t>(row) * K + k;
          topk_w[o] = renormalize ? bw[k] / wsum : bw[k];
          topk_ids[o] = bi[k];
          tok_exp_idx[o] = k * T + row;
        }
    }
  } else {
    for (int k = 0; k < K; ++k) {
      float best;
      int bidx;
      round(best, bidx);
      if (live && t == 0) {
        const size_t o = static_cast<size_t>(row) * K + k;
        topk_w[o] = best;
        topk_ids[o] = bidx;
        tok_exp_idx[o] = k * T + row;
      }
    }
    if (renormalize && live && t == 0) {
      for (int k = 0; k < K; ++k) {
        const size_t o = static_cast<size_t>(row) * K + k;
        topk_w[o] = topk_w[o] / wsum;
      }
    }
  }
}

}  // namespace
