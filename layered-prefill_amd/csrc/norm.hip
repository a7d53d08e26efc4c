// RMSNorm with the residual add in front of it: the step that feeds the MoE block
// (post_attention_layernorm in nanovllm/models/qwen3_moe.py, kernels
// csrc/layernorm_kernels.cu:10-35 and :77-108 of the reference).
//
//   s        = float(x) + float(residual)        (residual absent: s = float(x))
//   residual = T(s)
//   r        = rsqrt(mean(s^2) + eps)            (s before it is rounded, fp32)
//   out      = T( T(float(residual) * r) * weight )
//
// Bandwidth-bound: each element is read once and written once per tensor.  One
// wavefront owns one row; a lane holds its share of the row in registers (16-byte
// loads), so the rounded sums are never read back from memory, the reduction is
// a DPP/shuffle butterfly inside the wavefront and no LDS or barrier is needed.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerBlock = kThreads / kWave;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
  return v;
}

struct alignas(16) Pack8 {
  uint16_t v[8];
};

// 16-bit dtypes, H a multiple of 8 and at most 512 * NV, all rows 16-byte aligned.
template <typename El, int NV, bool ADD>
__global__ __launch_bounds__(kThreads) void rms_norm_vec_kernel(uint16_t* out, int64_t out_stride,
                                                                uint16_t* residual, int64_t res_stride,
                                                                const uint16_t* x, int64_t x_stride,
                                                                const uint16_t* __restrict__ weight, float eps,
                                                                int64_t T, int H) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = blockIdx.x * static_cast<int64_t>(kRowsPerBlock) + (threadIdx.x >> 6);
  if (row >= T) return;
  float s[NV][8];
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = (j * kWave + lane) * 8;
    if (c < H) {
      const Pack8 xv = *reinterpret_cast<const Pack8*>(x + row * x_stride + c);
      if constexpr (ADD) {
        const Pack8 rv = *reinterpret_cast<const Pack8*>(residual + row * res_stride + c);
        Pack8 ro;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float v = El::ld(xv.v[i]) + El::ld(rv.v[i]);
          sq += v * v;
          ro.v[i] = El::st(v);
          s[j][i] = El::ld(ro.v[i]);
        }
        *reinterpret_cast<Pack8*>(residual + row * res_stride + c) = ro;
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          s[j][i] = El::ld(xv.v[i]);
          sq += s[j][i] * s[j][i];
        }
      }
    }
  }
  const float r = rsqrtf(wave_sum(sq) / static_cast<float>(H) + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = (j * kWave + lane) * 8;
    if (c < H) {
      const Pack8 wv = *reinterpret_cast<const Pack8*>(weight + c);
      Pack8 o;
#pragma unroll
      for (int i = 0; i < 8; ++i) o.v[i] = El::st(El::ld(El::st(s[j][i] * r)) * El::ld(wv.v[i]));
      *reinterpret_cast<Pack8*>(out + row * out_stride + c) = o;
    }
  }
}

// Any dtype, size and alignment: two passes over the row, the second one reads
// back what this lane itself stored.
template <typename El, bool ADD>
__global__ __launch_bounds__(kThreads) void rms_norm_any_kernel(typename El::S* out, int64_t out_stride,
                                                                typename El::S* residual, int64_t res_stride,
                                                                const typename El::S* x, int64_t x_stride,
                                                                const typename El::S* __restrict__ weight, float eps,
                                                                int64_t T, int H) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = blockIdx.x * static_cast<int64_t>(kRowsPerBlock) + (threadIdx.x >> 6);
  if (row >= T) return;
  float sq = 0.f;
  for (int c = lane; c < H; c += kWave) {
    float v = El::ld(x[row * x_stride + c]);
    if constexpr (ADD) {
      v += El::ld(residual[row * res_stride + c]);
      residual[row * res_stride + c] = El::st(v);
    }
    sq += v * v;
  }
  const float r = rsqrtf(wave_sum(sq) / static_cast<float>(H) + eps);
  for (int c = lane; c < H; c += kWave) {
    const float v = ADD ? El::ld(residual[row * res_stride + c]) : El::ld(x[row * x_stride + c]);
    out[row * out_stride + c] = El::st(El::ld(El::st(v * r)) * El::ld(weight[c]));
  }
}

template <typename El, bool ADD>
int launch_norm(void* out, int64_t out_stride, void* residual, int64_t res_stride, const void* x,
                int64_t x_stride, const void* weight, float eps, int64_t T, int H, hipStream_t s) {
  using S = typename El::S;
  const int64_t blocks = (T + kRowsPerBlock - 1) / kRowsPerBlock;
  if (blocks > INT32_MAX) return moe_fail(MOE_ERR_ARG, "rms_norm: %lld rows", static_cast<long long>(T));
  const dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
  if constexpr (sizeof(S) == 2) {
    auto aligned = [](const void* p, int64_t stride) {
      return (reinterpret_cast<uintptr_t>(p) & 15u) == 0 && (stride & 7) == 0;
    };
    const bool vec = (H & 7) == 0 && H <= 512 * 16 && aligned(out, out_stride) && aligned(x, x_stride) &&
                     (!ADD || aligned(residual, res_stride)) && (reinterpret_cast<uintptr_t>(weight) & 15u) == 0;
    if (vec) {
      uint16_t* o = static_cast<uint16_t*>(out);
      uint16_t* r = static_cast<uint16_t*>(residual);
      const uint16_t* xi = static_cast<const uint16_t*>(x);
      const uint16_t* w = static_cast<const uint16_t*>(weight);
#define MOE_NORM_CASE(NV)                                                                                   \
  hipLaunchKernelGGL((rms_norm_vec_kernel<El, NV, ADD>), grid, block, 0, s, o, out_stride, r, res_stride, xi, \
                     x_stride, w, eps, T, H)
      if (H <= 512) MOE_NORM_CASE(1);
      else if (H <= 1024) MOE_NORM_CASE(2);
      else if (H <= 2048) MOE_NORM_CASE(4);
      else if (H <= 4096) MOE_NORM_CASE(8);
      else MOE_NORM_CASE(16);
#undef MOE_NORM_CASE
      return moe_check_launch(ADD ? "add_rms_norm" : "rms_norm");
    }
  }
  hipLaunchKernelGGL((rms_norm_any_kernel<El, ADD>), grid, block, 0, s, static_cast<S*>(out), out_stride,
                     static_cast<S*>(residual), res_stride, static_cast<const S*>(x), x_stride,
                     static_cast<const S*>(weight), eps, T, H);
  return moe_check_launch(ADD ? "add_rms_norm" : "rms_norm");
}

}  // namespace

MOE_EXPORT int moe_add_rms_norm(void* out, int64_t out_stride, void* residual, int64_t residual_stride,
                                const void* x, int64_t x_stride, const void* weight, int dtype, int64_t T,
                                int H, float eps, void* stream) {
  if (T < 0 || H < 1) return moe_fail(MOE_ERR_ARG, "rms_norm: bad sizes T=%lld H=%d", static_cast<long long>(T), H);
  if (T == 0) return MOE_OK;
  if (!out || !x || !weight) return moe_fail(MOE_ERR_ARG, "rms_norm: null tensor pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
#define MOE_NORM_DTYPE(El)                                                                                        \
  return residual ? launch_norm<El, true>(out, out_stride, residual, residual_stride, x, x_stride, weight, eps, T, H, s) \
                  : launch_norm<El, false>(out, out_stride, nullptr, 0, x, x_stride, weight, eps, T, H, s)
  switch (dtype) {
    case MOE_BF16: MOE_NORM_DTYPE(ElemBF16);
    case MOE_F16: MOE_NORM_DTYPE(ElemF16);
    case MOE_F32: MOE_NORM_DTYPE(ElemF32);
    default: return moe_fail(MOE_ERR_UNSUPPORTED, "rms_norm: dtype code %d", dtype);
  }
#undef MOE_NORM_DTYPE
}
