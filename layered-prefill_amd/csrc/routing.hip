// Router: row softmax over E experts + K rounds of argmax, one launch.
//
// Replaces topkGatingSoftmax / moeSoftmax + moeTopK of the reference
// (csrc/moe_topk_softmax_kernels.cu:50-166,182-380, dispatch :421-471).
// For power-of-two E <= 256 a row is shared by the same number of lanes, with
// the same column-to-lane assignment and the same butterfly order, as in the
// reference's fused kernel, so the fp32 sum has the same association; the
// 64-lane wavefront simply carries twice as many rows as a 32-lane warp.
// Any other E <= 1024 takes one wavefront per row.
#include <stdarg.h>

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
constexpr float kFltMin = 1.17549435e-38f;

template <int E>
__global__ __launch_bounds__(kWave* kWavesPerBlock) void topk_softmax_pow2_kernel(
    const float* __restrict__ gating, float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
    int32_t* __restrict__ tok_exp_idx, int T, int K, int renormalize) {
  using G = Pow2Geom<E>;
  constexpr int EPL = G::kEpl, VECS = G::kVecs, VPT = G::kVpt, TPR = G::kTpr;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int row = (blockIdx.x * kWavesPerBlock + wave) * G::kRowsPerWave + lane / TPR;
  const int t = lane % TPR;
  const bool live = row < T;
  const int ld_row = live ? row : (T - 1);

  float v[VPT];
  const float* src = gating + static_cast<size_t>(ld_row) * E + t * EPL;
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

  float mx = v[0];
#pragma unroll
  for (int i = 1; i < VPT; ++i) mx = fmaxf(mx, v[i]);
#pragma unroll
  for (int m = TPR / 2; m > 0; m /= 2) mx = fmaxf(mx, __shfl_xor(mx, m, kWave));

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
  for (int i = 0; i < VPT; ++i) {
    float p = v[i] * rinv;
    v[i] = p < kFltMin ? 0.f : p;
  }

  // Up to kRegK winners stay in registers until the row is done, so that the
  // renormalised weights are written once (reading the stored weights back
  // would wait for the stores to complete).
  constexpr int kRegK = 16;
  float wsum = 0.f;
  float bw[kRegK];
#pragma unroll
  for (int k = 0; k < kRegK; ++k) bw[k] = 0.f;
  auto round = [&](int k, float& best_out) {
    float best = v[0];
    int bidx = t * EPL;
#pragma unroll
    for (int i = 1; i < VPT; ++i) {
      const int col = (i / EPL) * (EPL * TPR) + t * EPL + (i % EPL);
      if (v[i] > best) { best = v[i]; bidx = col; }
    }
#pragma unroll
    for (int m = TPR / 2; m > 0; m /= 2) {
      float ov = __shfl_xor(best, m, kWave);
      int oi = __shfl_xor(bidx, m, kWave);
      if (ov > best || (ov == best && oi < bidx)) { best = ov; bidx = oi; }
    }
    if (live && t == 0) {
      const size_t o = static_cast<size_t>(row) * K + k;
      topk_ids[o] = bidx;
      tok_exp_idx[o] = k * T + row;
    }
    wsum += best;
    best_out = best;
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
      if (k < K) round(k, bw[k]);
    if (live && t == 0) {
#pragma unroll
      for (int k = 0; k < kRegK; ++k)
        if (k < K) topk_w[static_cast<size_t>(row) * K + k] = renormalize ? bw[k] / wsum : bw[k];
    }
  } else {
    for (int k = 0; k < K; ++k) {
      float best;
      round(k, best);
      if (live && t == 0) topk_w[static_cast<size_t>(row) * K + k] = best;
    }
    if (renormalize && live && t == 0) {
      for (int k = 0; k < K; ++k) {
        const size_t o = static_cast<size_t>(row) * K + k;
        topk_w[o] = topk_w[o] / wsum;
      }
    }
  }
}

// One wavefront per row; lane l holds columns l, l+64, ... (up to 16 of them).
constexpr int kGenericMaxPerLane = 16;

__global__ __launch_bounds__(kWave* kWavesPerBlock) void topk_softmax_generic_kernel(
    const float* __restrict__ gating, float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
    int32_t* __restrict__ tok_exp_idx, int T, int E, int K, int renormalize) {
  const int lane = threadIdx.x % kWave;
  const int row = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  const bool live = row < T;
  const float* src = gating + static_cast<size_t>(live ? row : T - 1) * E;
  const float ninf = -__builtin_inff();

  float v[kGenericMaxPerLane];
  float mx = ninf;
#pragma unroll
  for (int j = 0; j < kGenericMaxPerLane; ++j) {
    const int c = lane + j * kWave;
    v[j] = c < E ? src[c] : ninf;
    mx = fmaxf(mx, v[j]);
  }
#pragma unroll
  for (int m = 32; m > 0; m /= 2) mx = fmaxf(mx, __shfl_xor(mx, m, kWave));
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < kGenericMaxPerLane; ++j) {
    const int c = lane + j * kWave;
    if (c < E) {
      v[j] = moe_expf(v[j] - mx);
      sum += v[j];
    }
  }
#pragma unroll
  for (int m = 32; m > 0; m /= 2) sum += __shfl_xor(sum, m, kWave);
  const float rinv = 1.f / sum;
#pragma unroll
  for (int j = 0; j < kGenericMaxPerLane; ++j) {
    const int c = lane + j * kWave;
    float p = v[j] * rinv;
    p = p < kFltMin ? 0.f : p;
    v[j] = c < E ? p : -20000.f;  // columns past E can never win
  }

  float wsum = 0.f;
  for (int k = 0; k < K; ++k) {
    float best = v[0];
    int bidx = lane;
#pragma unroll
    for (int j = 1; j < kGenericMaxPerLane; ++j)
      if (v[j] > best) { best = v[j]; bidx = lane + j * kWave; }
#pragma unroll
    for (int m = 32; m > 0; m /= 2) {
      float ov = __shfl_xor(best, m, kWave);
      int oi = __shfl_xor(bidx, m, kWave);
      if (ov > best || (ov == best && oi < bidx)) { best = ov; bidx = oi; }
    }
    if (live && lane == 0) {
      const size_t o = static_cast<size_t>(row) * K + k;
      topk_w[o] = best;
      topk_ids[o] = bidx;
      tok_exp_idx[o] = k * T + row;
    }
    wsum += best;
#pragma unroll
    for (int j = 0; j < kGenericMaxPerLane; ++j)
      if (lane == bidx % kWave && j == bidx / kWave) v[j] = -10000.f;
  }
  if (renormalize && live && lane == 0) {
    for (int k = 0; k < K; ++k) {
      const size_t o = static_cast<size_t>(row) * K + k;
      topk_w[o] = topk_w[o] / wsum;
    }
  }
}

template <int E>
void launch_pow2(const float* g, float* w, int32_t* ids, int32_t* tei, int T, int K, int renorm,
                 hipStream_t s) {
  constexpr int rows_per_block = Pow2Geom<E>::kRowsPerWave * kWavesPerBlock;
  const int blocks = (T + rows_per_block - 1) / rows_per_block;
  hipLaunchKernelGGL(topk_softmax_pow2_kernel<E>, dim3(blocks), dim3(kWave * kWavesPerBlock), 0, s,
                     g, w, ids, tei, T, K, renorm);
}

}  // namespace

MOE_EXPORT int moe_topk_softmax(const float* gating_output, float* topk_weights, int32_t* topk_ids,
                                int32_t* token_expert_indices, int T, int E, int K,
                                int renormalize, void* stream) {
  if (T < 0 || E < 1 || K < 1) return moe_fail(MOE_ERR_ARG, "topk_softmax: bad sizes T=%d E=%d K=%d", T, E, K);
  if (K > E) return moe_fail(MOE_ERR_ARG, "topk_softmax: topk %d exceeds num_experts %d", K, E);
  if (E > kWave * kGenericMaxPerLane)
    return moe_fail(MOE_ERR_UNSUPPORTED, "topk_softmax: num_experts %d > %d", E, kWave * kGenericMaxPerLane);
  if (static_cast<int64_t>(T) * K > INT32_MAX)
    return moe_fail(MOE_ERR_ARG, "topk_softmax: T*K overflows int32 token_expert_indices");
  if (T == 0) return MOE_OK;
  if (!gating_output || !topk_weights || !topk_ids || !token_expert_indices)
    return moe_fail(MOE_ERR_ARG, "topk_softmax: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (E) {
    case 1: launch_pow2<1>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    case 2: launch_pow2<2>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    case 4: launch_pow2<4>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    case 8: launch_pow2<8>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    case 16: launch_pow2<16>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    case 32: launch_pow2<32>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    case 64: launch_pow2<64>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    case 128: launch_pow2<128>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    case 256: launch_pow2<256>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, s); break;
    default: {
      const int blocks = (T + kWavesPerBlock - 1) / kWavesPerBlock;
      hipLaunchKernelGGL(topk_softmax_generic_kernel, dim3(blocks), dim3(kWave * kWavesPerBlock), 0,
                         s, gating_output, topk_weights, topk_ids, token_expert_indices, T, E, K,
                         renormalize);
    }
  }
  return moe_check_launch("topk_softmax");
}
