// Router: row softmax over E experts + K rounds of argmax, one launch.
//
// Replaces topkGatingSoftmax / moeSoftmax + moeTopK of the reference
// (csrc/moe_topk_softmax_kernels.cu:50-166,182-380, dispatch :421-471).
// For power-of-two E <= 256 a row is shared by the same number of lanes, with
// the same column-to-lane assignment and the same butterfly order, as in the
// reference's fused kernel, so the fp32 sum has the same association; the
// 64-lane wavefront simply carries twice as many rows as a 32-lane warp.
// Any other E takes one wavefront per row: in registers up to 1024 columns, in LDS up to 16384.
#include <stdarg.h>

#include "common.h"
#include "routing_device.h"

namespace {

template <int E>
__global__ __launch_bounds__(kWave* kWavesPerBlock) void topk_softmax_pow2_kernel(
    const float* __restrict__ gating, float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
    int32_t* __restrict__ tok_exp_idx, int T, int K, int renormalize) {
  using G = Pow2Geom<E>;
  constexpr int VPT = G::kVpt, TPR = G::kTpr;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int row = (blockIdx.x * kWavesPerBlock + wave) * G::kRowsPerWave + lane / TPR;
  const int t = lane % TPR;
  const bool live = row < T;
  const int ld_row = live ? row : (T - 1);

  float v[VPT];
  load_row<E>(gating, ld_row, t, v);
  route_row<E>(v, t, row, live, topk_w, topk_ids, tok_exp_idx, T, K, renormalize);
}

// ---------------------------------------------------------------------------
// Router gate fused in front: logits = x . Wg^T (the reference's ReplicatedLinear,
// nanovllm/models/qwen3_moe.py:93-104, whose output has the activation dtype),
// rounded to that dtype, then the same softmax / top-k as above, without the
// logits ever leaving the CU.  A workgroup takes 32 tokens and all E experts
// and walks K in units of 64 elements: the unit's 32 token rows and E gate rows
// (128 bytes each) go global->LDS by DMA into a ring of four units, full
// 128-byte lines per request (operands fetched straight into MFMA register
// layout touch 64 different lines per wavefront load and ran 3x slower than the
// separate GEMM + routing kernels).  Wavefront f multiplies expert fragment f
// (MFMA 32x32x16, experts as the A operand, tokens as B); the rounded logits
// are laid out in LDS as [token][expert] and routed from there with the lane
// layout of the stand-alone kernel.
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 gate_bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 gate_f16x8;
typedef __attribute__((ext_vector_type(16))) float gate_f32x16;
typedef __attribute__((address_space(3))) char gate_lds_char;

template <typename El>
__device__ __forceinline__ gate_f32x16 gate_mma(const uint4& a, const uint4& b, gate_f32x16 c);
template <>
__device__ __forceinline__ gate_f32x16 gate_mma<ElemBF16>(const uint4& a, const uint4& b, gate_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(gate_bf16x8, a),
                                                 __builtin_bit_cast(gate_bf16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ gate_f32x16 gate_mma<ElemF16>(const uint4& a, const uint4& b, gate_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(gate_f16x8, a),
                                                __builtin_bit_cast(gate_f16x8, b), c, 0, 0, 0);
}

// 16 bytes per lane from global memory straight into LDS at lds_wave_base + 16 * lane
// (issued from assembly: the compiler would order every later LDS read behind it with vmcnt(0))
__device__ __forceinline__ void gate_dma16(const char* base, uint32_t lane_byte_offset, uint32_t lds_wave_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(lds_wave_base), "v"(lane_byte_offset), "s"(base)
      : "memory");
}

constexpr int kGateTokens = 32, kGateRowBytes = 128;

constexpr int kGateWaves = 16;  // wavefronts 0..3 stream and multiply; all sixteen route (two rows each)

template <typename El, int E, int kGateRing>
__global__ __launch_bounds__(kWave* kGateWaves) void gate_topk_softmax_kernel(
    const typename El::S* __restrict__ x, const typename El::S* __restrict__ wg,
    float* __restrict__ logits_out, float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
    int32_t* __restrict__ tok_exp_idx, int T, int H, int K, int renormalize) {
  using G = Pow2Geom<E>;
  constexpr int NF = E / 32;                         // expert fragments = computing wavefronts
  constexpr int WJ = E / 32;                         // gate-row requests per wavefront and unit
  constexpr int kWBytes = E * kGateRowBytes;
  constexpr int kUnitBytes = kWBytes + kGateTokens * kGateRowBytes;
  constexpr int kDma = WJ + 1;                       // requests per wavefront and unit
  static_assert(NF >= 1 && NF <= kWavesPerBlock, "one expert fragment per wavefront");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int l32 = lane & 31, lhi = lane >> 5;
  const int t0 = blockIdx.x * kGateTokens;

  // DMA: a request covers 8 rows x 128 bytes; lane / 8 is the row, lane % 8 the 16-byte chunk
  // it lands in; chunk c of row r holds logical chunk c ^ ((r >> 1) & 7) (bank spreading)
  const int q = lane >> 3;
  uint32_t a_off, w_off[WJ];
  {
    const int rr = 8 * wave + q;
    const int row = t0 + rr < T ? t0 + rr : T - 1;
    a_off = static_cast<uint32_t>(static_cast<size_t>(row) * H * 2 + (((lane & 7) ^ ((rr >> 1) & 7)) << 4));
  }
#pragma unroll
  for (int j = 0; j < WJ; ++j) {
    const int rr = (E / 4) * wave + 8 * j + q;
    w_off[j] = static_cast<uint32_t>(static_cast<size_t>(rr) * H * 2 + (((lane & 7) ^ ((rr >> 1) & 7)) << 4));
  }
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const gate_lds_char*)smem));
  const uint32_t dma_w = __builtin_amdgcn_readfirstlane(lds0 + (E / 4) * wave * kGateRowBytes);
  const uint32_t dma_a = __builtin_amdgcn_readfirstlane(lds0 + kWBytes + 8 * wave * kGateRowBytes);
  const char* xb = reinterpret_cast<const char*>(x);
  const char* wb = reinterpret_cast<const char*>(wg);
  const bool worker = wave < kWavesPerBlock;  // the other wavefronts only keep the barriers company
  auto issue = [&](int u) {
    if (!worker) return;
    const uint32_t ring = (u % kGateRing) * kUnitBytes;
    gate_dma16(xb + u * kGateRowBytes, a_off, dma_a + ring);
#pragma unroll
    for (int j = 0; j < WJ; ++j) gate_dma16(wb + u * kGateRowBytes, w_off[j], dma_w + ring + j * 1024);
  };
  int rd_k[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) rd_k[kk] = l32 * kGateRowBytes + (((2 * kk + lhi) ^ ((l32 >> 1) & 7)) << 4);

  gate_f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  const int nu = H / 64;
  constexpr int AHEAD = kGateRing - 1;  // units in flight
#pragma unroll
  for (int u = 0; u < AHEAD; ++u)
    if (u < nu) issue(u);
  for (int u = 0; u < nu; ++u) {
    // unit u has landed (only the AHEAD-1 younger units may be outstanding; near the end
    // fewer are, and waiting for all of them is as good); everybody has left unit u-1
    if (u + AHEAD - 1 < nu) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((AHEAD - 1) * kDma) : "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    asm volatile("s_barrier" ::: "memory");
    if (u + AHEAD < nu) issue(u + AHEAD);
    if (worker && wave < NF) {
      const char* st = smem + (u % kGateRing) * kUnitBytes;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const uint4 xf = *reinterpret_cast<const uint4*>(st + kWBytes + rd_k[kk]);
        const uint4 wf = *reinterpret_cast<const uint4*>(st + wave * 32 * kGateRowBytes + rd_k[kk]);
        acc = gate_mma<El>(wf, xf, acc);
      }
    }
  }
  __syncthreads();  // the ring is free: it now holds the logits, [token][expert] fp32
  float* lg = reinterpret_cast<float*>(smem);
  if (worker && wave < NF) {
    // acc[r]: expert 32 wave + 8 (r / 4) + 4 lhi + r % 4, token l32; one rounding to the activation dtype
#pragma unroll
    for (int r = 0; r < 16; ++r)
      lg[l32 * E + wave * 32 + 8 * (r / 4) + 4 * lhi + (r % 4)] = El::ld(El::st(acc[r]));
  }
  __syncthreads();
  if (logits_out) {
    for (int i = threadIdx.x; i < kGateTokens * E; i += kWave * kGateWaves) {
      const int row = t0 + i / E;
      if (row < T) logits_out[static_cast<size_t>(row) * E + i % E] = lg[i];
    }
  }
  // routing, rows in the stand-alone kernel's lane layout
  constexpr int EPL = G::kEpl, VECS = G::kVecs, VPT = G::kVpt, TPR = G::kTpr, RPW = G::kRowsPerWave;
  const int t = lane % TPR;
  for (int r0 = wave * RPW; r0 < kGateTokens; r0 += kGateWaves * RPW) {
    const int lrow = r0 + lane / TPR;
    const int row = t0 + lrow;
    float v[VPT];
#pragma unroll
    for (int j = 0; j < VECS; ++j)
#pragma unroll
      for (int i = 0; i < EPL; ++i) v[j * EPL + i] = lg[lrow * E + j * EPL * TPR + t * EPL + i];
    route_row<E>(v, t, row, row < T, topk_w, topk_ids, tok_exp_idx, T, K, renormalize);
  }
}

template <typename El, int E>
int launch_gate(const void* x, const void* wg, float* logits_out, float* w, int32_t* ids,
                 int32_t* tei, int T, int H, int K, int renorm, hipStream_t s) {
  using S = typename El::S;
  const int blocks = (T + kGateTokens - 1) / kGateTokens;
  // few workgroups (decode): one per CU with a deep ring, 140 KB at E = 128; many: two per CU, 80 KB
  if (blocks <= 256) {
    constexpr int lds = 7 * (E + kGateTokens) * kGateRowBytes;
    auto kern = gate_topk_softmax_kernel<El, E, 7>;
    static MoeLdsOptIn opted;
    if (int rc = moe_opt_in_lds(opted, reinterpret_cast<const void*>(kern), lds, "gate_topk_softmax")) return rc;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(kWave * kGateWaves), lds, s,
                       static_cast<const S*>(x), static_cast<const S*>(wg), logits_out, w, ids, tei, T, H, K, renorm);
  } else {
    constexpr int lds = 4 * (E + kGateTokens) * kGateRowBytes;
    auto kern = gate_topk_softmax_kernel<El, E, 4>;
    static MoeLdsOptIn opted;
    if (int rc = moe_opt_in_lds(opted, reinterpret_cast<const void*>(kern), lds, "gate_topk_softmax")) return rc;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(kWave * kGateWaves), lds, s,
                       static_cast<const S*>(x), static_cast<const S*>(wg), logits_out, w, ids, tei, T, H, K, renorm);
  }
  return MOE_OK;
}

template <typename El>
int launch_gate_e(const void* x, const void* wg, float* logits_out, float* w, int32_t* ids,
                  int32_t* tei, int T, int H, int E, int K, int renorm, hipStream_t s) {
  switch (E) {
    case 32: if (int rc = launch_gate<El, 32>(x, wg, logits_out, w, ids, tei, T, H, K, renorm, s)) return rc; break;
    case 64: if (int rc = launch_gate<El, 64>(x, wg, logits_out, w, ids, tei, T, H, K, renorm, s)) return rc; break;
    case 128: if (int rc = launch_gate<El, 128>(x, wg, logits_out, w, ids, tei, T, H, K, renorm, s)) return rc; break;
    default: return moe_fail(MOE_ERR_UNSUPPORTED, "gate_topk_softmax: num_experts %d (32, 64 or 128)", E);
  }
  return moe_check_launch("gate_topk_softmax");
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
    const float p = v[j] * rinv;
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

// Wider rows (more columns than 64 lanes x 16 registers): one wavefront per row,
// the row's probabilities in LDS.  Lane l owns columns l, l+64, ... exactly as in
// the register kernel above, so the order of every max, sum and comparison is the
// same; every LDS word is read and written by its owning lane only, which is why
// no barrier appears.
constexpr int kWideMaxExperts = 16384;  // 64 KiB of LDS per row

__global__ __launch_bounds__(kWave) void topk_softmax_wide_kernel(
    const float* __restrict__ gating, float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
    int32_t* __restrict__ tok_exp_idx, int T, int E, int K, int renormalize) {
  extern __shared__ float prob[];
  const int lane = threadIdx.x;
  const int row = blockIdx.x;
  const float* src = gating + static_cast<size_t>(row) * E;
  const float ninf = -__builtin_inff();

  float mx = ninf;
  for (int c = lane; c < E; c += kWave) mx = fmaxf(mx, src[c]);
#pragma unroll
  for (int m = 32; m > 0; m /= 2) mx = fmaxf(mx, __shfl_xor(mx, m, kWave));
  float sum = 0.f;
  for (int c = lane; c < E; c += kWave) {
    const float e = moe_expf(src[c] - mx);
    prob[c] = e;
    sum += e;
  }
#pragma unroll
  for (int m = 32; m > 0; m /= 2) sum += __shfl_xor(sum, m, kWave);
  const float rinv = 1.f / sum;
  for (int c = lane; c < E; c += kWave) prob[c] = prob[c] * rinv;

  float wsum = 0.f;
  for (int k = 0; k < K; ++k) {
    // below the marker of a taken column.  (A row with fewer than K comparable probabilities, i.e.
    // NaN logits, lets a taken column win again: the reference's fallback kernel behaves the same,
    // csrc/moe_topk_softmax_kernels.cu:117-150, and such rows carry no meaning.)
    float best = -20000.f;
    int bidx = lane;
    for (int c = lane; c < E; c += kWave) {
      const float v = prob[c];
      if (v > best) { best = v; bidx = c; }
    }
#pragma unroll
    for (int m = 32; m > 0; m /= 2) {
      float ov = __shfl_xor(best, m, kWave);
      int oi = __shfl_xor(bidx, m, kWave);
      if (ov > best || (ov == best && oi < bidx)) { best = ov; bidx = oi; }
    }
    if (lane == 0) {
      const size_t o = static_cast<size_t>(row) * K + k;
      topk_w[o] = best;
      topk_ids[o] = bidx;
      tok_exp_idx[o] = k * T + row;
    }
    wsum += best;
    if (lane == bidx % kWave) prob[bidx] = -10000.f;
  }
  if (renormalize && lane == 0) {
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
  if (E > kWideMaxExperts)
    return moe_fail(MOE_ERR_UNSUPPORTED, "topk_softmax: num_experts %d > %d", E, kWideMaxExperts);
  if (static_cast<int64_t>(T) * K > INT32_MAX)
    return moe_fail(MOE_ERR_ARG, "topk_softmax: T*K overflows int32 token_expert_indices");
  // one 64-lane workgroup per row beyond 1024 experts: the grid's thread count has to fit 32 bits
  if (E > kWave * kGenericMaxPerLane && static_cast<int64_t>(T) > (static_cast<int64_t>(UINT32_MAX) / kWave))
    return moe_fail(MOE_ERR_UNSUPPORTED, "topk_softmax: %d rows of %d experts exceed the launch limit of %lld rows", T, E,
                    static_cast<long long>(UINT32_MAX / kWave));
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
      if (E > kWave * kGenericMaxPerLane) {
        hipLaunchKernelGGL(topk_softmax_wide_kernel, dim3(T), dim3(kWave), sizeof(float) * E, s,
                           gating_output, topk_weights, topk_ids, token_expert_indices, T, E, K,
                           renormalize);
        break;
      }
      const int blocks = (T + kWavesPerBlock - 1) / kWavesPerBlock;
      hipLaunchKernelGGL(topk_softmax_generic_kernel, dim3(blocks), dim3(kWave * kWavesPerBlock), 0,
                         s, gating_output, topk_weights, topk_ids, token_expert_indices, T, E, K,
                         renormalize);
    }
  }
  return moe_check_launch("topk_softmax");
}

MOE_EXPORT int moe_gate_topk_softmax(const void* x, const void* gate_weight, int dtype,
                                     float* logits_out, float* topk_weights, int32_t* topk_ids,
                                     int32_t* token_expert_indices, int T, int H, int E, int K,
                                     int renormalize, void* stream) {
  if (T < 0 || H < 1 || E < 1 || K < 1) return moe_fail(MOE_ERR_ARG, "gate_topk_softmax: bad sizes T=%d H=%d E=%d K=%d", T, H, E, K);
  if (K > E) return moe_fail(MOE_ERR_ARG, "gate_topk_softmax: topk %d exceeds num_experts %d", K, E);
  if (static_cast<int64_t>(T) * K > INT32_MAX)
    return moe_fail(MOE_ERR_ARG, "gate_topk_softmax: T*K overflows int32 token_expert_indices");
  if (H % 64 != 0)
    return moe_fail(MOE_ERR_UNSUPPORTED, "gate_topk_softmax: hidden size %d is not a multiple of 64", H);
  if (static_cast<int64_t>(T) * H * 2 >= (1LL << 32))
    return moe_fail(MOE_ERR_UNSUPPORTED, "gate_topk_softmax: x larger than 4 GiB (32-bit row offsets)");
  if (T == 0) return MOE_OK;
  if (!x || !gate_weight || !topk_weights || !topk_ids || !token_expert_indices)
    return moe_fail(MOE_ERR_ARG, "gate_topk_softmax: null pointer");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gate_weight)) & 15u)
    return moe_fail(MOE_ERR_ARG, "gate_topk_softmax: x and the gate weight must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MOE_BF16: return launch_gate_e<ElemBF16>(x, gate_weight, logits_out, topk_weights, topk_ids, token_expert_indices, T, H, E, K, renormalize, s);
    case MOE_F16: return launch_gate_e<ElemF16>(x, gate_weight, logits_out, topk_weights, topk_ids, token_expert_indices, T, H, E, K, renormalize, s);
    default: return moe_fail(MOE_ERR_UNSUPPORTED, "gate_topk_softmax: dtype code %d (bf16 or fp16)", dtype);
  }
}
