// Bandwidth-bound helpers of the expert path: the stand-alone gated
// activations (csrc/activation_kernels.cu:14-64 of the reference), the top-k
// combine (nanovllm/layers/for_moe/moe_easy_kernel.py:26-31) and fp8 row
// quantisation.  16-byte vector accesses, grid-stride loops.
#include "common.h"

namespace {

constexpr int kThreads = 256;

template <typename S, int N>
struct alignas(sizeof(S) * N) Vec {
  S v[N];
};

// out[r, i] = T(silu(in[r, i])) * in[r, d + i]; the product is taken in T.
template <typename El, int VEC>
__global__ __launch_bounds__(kThreads) void silu_and_mul_kernel(typename El::S* __restrict__ out,
                                                                const typename El::S* __restrict__ in,
                                                                int64_t rows, int d) {
  using S = typename El::S;
  const int per_row = d / VEC;
  const int64_t total = rows * per_row;
  for (int64_t idx = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x; idx < total;
       idx += static_cast<int64_t>(gridDim.x) * kThreads) {
    const int64_t r = idx / per_row;
    const int c = static_cast<int>(idx - r * per_row) * VEC;
    const Vec<S, VEC> g = *reinterpret_cast<const Vec<S, VEC>*>(in + r * 2 * d + c);
    const Vec<S, VEC> u = *reinterpret_cast<const Vec<S, VEC>*>(in + r * 2 * d + d + c);
    Vec<S, VEC> o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float s = El::ld(El::st(moe_silu(El::ld(g.v[i]))));
      o.v[i] = El::st(s * El::ld(u.v[i]));
    }
    *reinterpret_cast<Vec<S, VEC>*>(out + r * d + c) = o;
  }
}

// out[r, i] = T(swigluoai(in[r, 2i], in[r, 2i+1]))
template <typename El, int VEC>
__global__ __launch_bounds__(kThreads) void swigluoai_and_mul_kernel(
    typename El::S* __restrict__ out, const typename El::S* __restrict__ in, int64_t rows, int d,
    float alpha, float limit) {
  using S = typename El::S;
  const int per_row = d / VEC;
  const int64_t total = rows * per_row;
  for (int64_t idx = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x; idx < total;
       idx += static_cast<int64_t>(gridDim.x) * kThreads) {
    const int64_t r = idx / per_row;
    const int c = static_cast<int>(idx - r * per_row) * VEC;
    const Vec<S, 2 * VEC> x = *reinterpret_cast<const Vec<S, 2 * VEC>*>(in + r * 2 * d + 2 * c);
    Vec<S, VEC> o;
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      o.v[i] = El::st(moe_swigluoai(El::ld(x.v[2 * i]), El::ld(x.v[2 * i + 1]), alpha, limit));
    *reinterpret_cast<Vec<S, VEC>*>(out + r * d + c) = o;
  }
}

// out[t, h] = sum_k in[t, k, h], ascending k, fp32 accumulation.
template <typename El, int VEC>
__global__ __launch_bounds__(kThreads) void moe_sum_kernel(typename El::S* __restrict__ out,
                                                           const typename El::S* __restrict__ in,
                                                           int64_t T, int K, int H) {
  using S = typename El::S;
  const int per_row = H / VEC;
  const int64_t total = T * per_row;
  for (int64_t idx = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x; idx < total;
       idx += static_cast<int64_t>(gridDim.x) * kThreads) {
    const int64_t t = idx / per_row;
    const int c = static_cast<int>(idx - t * per_row) * VEC;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    for (int k = 0; k < K; ++k) {
      const Vec<S, VEC> x =
          *reinterpret_cast<const Vec<S, VEC>*>(in + (t * K + k) * static_cast<int64_t>(H) + c);
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] += El::ld(x.v[i]);
    }
    Vec<S, VEC> o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) o.v[i] = El::st(acc[i]);
    *reinterpret_cast<Vec<S, VEC>*>(out + t * static_cast<int64_t>(H) + c) = o;
  }
}


// fp32 -> OCP e4m3fn code, saturating at +-448, round to nearest even
// (v_cvt_pk_fp8_f32 on gfx950 produces the OCP encoding).
__device__ __forceinline__ uint8_t f32_to_e4m3(float v) {
  v = fminf(fmaxf(v, -448.f), 448.f);
  return static_cast<uint8_t>(__builtin_amdgcn_cvt_pk_fp8_f32(v, v, 0, false) & 0xff);
}

// Two values at once: bits 0-7 the code of a, bits 8-15 the code of b.
__device__ __forceinline__ uint32_t f32x2_to_e4m3(float a, float b) {
  a = __builtin_amdgcn_fmed3f(a, -448.f, 448.f);
  b = __builtin_amdgcn_fmed3f(b, -448.f, 448.f);
  return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false)) & 0xffffu;
}

// Smallest row scale: a row whose largest magnitude is tiny but not zero would get
// a scale whose reciprocal overflows (amax below about 1.3e-36); from 2^-100 down
// the scale stays 2^-100 and the row's codes are simply small.
constexpr float kMinScale = 7.888609052210118e-31f;  // 2^-100

// One wavefront per row: s = max(amax|row| / 448, 2^-100) (1 for an all-zero row),
// q = e4m3(row * (1 / s)): one correctly rounded division per row, then one
// multiplication per element (a division per element made the kernel
// VALU-bound: 48 us for 67584 x 768 against 28 us of memory time).
template <typename El>
__global__ __launch_bounds__(kThreads) void quant_rows_e4m3_kernel(
    const typename El::S* __restrict__ w, int64_t rows, int cols, uint8_t* __restrict__ q,
    float* __restrict__ scales, const int32_t* __restrict__ row_ids, int64_t id_count, int numel) {
  const int lane = threadIdx.x % kWave;
  const int64_t row = blockIdx.x * static_cast<int64_t>(kThreads / kWave) + threadIdx.x / kWave;
  if (row >= rows) return;
  if (row_ids && (row >= id_count || row_ids[row] >= numel)) return;  // a padding slot: nobody reads it
  const typename El::S* src = w + row * cols;
  float amax = 0.f;
  for (int c = lane; c < cols; c += kWave) amax = fmaxf(amax, fabsf(El::ld(src[c])));
#pragma unroll
  for (int m = 32; m > 0; m /= 2) amax = fmaxf(amax, __shfl_xor(amax, m, kWave));
  const float s = amax > 0.f ? fmaxf(amax / 448.f, kMinScale) : 1.f;
  if (lane == 0) scales[row] = s;
  const float inv = 1.0f / s;
  for (int c = lane; c < cols; c += kWave) q[row * cols + c] = f32_to_e4m3(El::ld(src[c]) * inv);
}

// 16-bit sources with up to NV * 512 columns: the row stays in registers between
// the amax pass and the conversion, 16 bytes in and 8 bytes out per lane and
// step.  Same arithmetic as the kernel above, element by element.
template <typename El, int NV>
__global__ __launch_bounds__(kThreads) void quant_rows_e4m3_vec_kernel(
    const typename El::S* __restrict__ w, int64_t rows, int cols, uint8_t* __restrict__ q,
    float* __restrict__ scales, const int32_t* __restrict__ row_ids, int64_t id_count, int numel) {
  const int lane = threadIdx.x % kWave;
  const int64_t row = blockIdx.x * static_cast<int64_t>(kThreads / kWave) + threadIdx.x / kWave;
  if (row >= rows) return;
  if (row_ids && (row >= id_count || row_ids[row] >= numel)) return;  // a padding slot: nobody reads it
  const uint4* src = reinterpret_cast<const uint4*>(w + row * cols);
  const int nvec = cols / 8;
  uint4 v[NV];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * kWave;
    v[i] = c < nvec ? src[c] : uint4{0, 0, 0, 0};
    const uint32_t wds[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      amax = fmaxf(amax, fabsf(El::ld(static_cast<uint16_t>(wds[j]))));
      amax = fmaxf(amax, fabsf(El::ld(static_cast<uint16_t>(wds[j] >> 16))));
    }
  }
#pragma unroll
  for (int m = 32; m > 0; m /= 2) amax = fmaxf(amax, __shfl_xor(amax, m, kWave));
  const float s = amax > 0.f ? fmaxf(amax / 448.f, kMinScale) : 1.f;
  if (lane == 0) scales[row] = s;
  const float inv = 1.0f / s;
  uint2* dst = reinterpret_cast<uint2*>(q + row * cols);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * kWave;
    if (c >= nvec) continue;
    const uint32_t wds[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
    uint32_t o[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      o[j >> 1] |= f32x2_to_e4m3(El::ld(static_cast<uint16_t>(wds[j])) * inv,
                                 El::ld(static_cast<uint16_t>(wds[j] >> 16)) * inv)
                   << (16 * (j & 1));
    dst[c] = uint2{o[0], o[1]};
  }
}

template <typename El>
bool launch_quant_vec(const void* w, int64_t rows, int cols, uint8_t* q, float* scales,
                      const int32_t* row_ids, int64_t id_count, int numel, dim3 grid, hipStream_t s) {
  using S = typename El::S;
  if (cols % 8 != 0 || cols > 4096 || (reinterpret_cast<uintptr_t>(w) & 15u) || (reinterpret_cast<uintptr_t>(q) & 7u))
    return false;
  const int nv = (cols / 8 + kWave - 1) / kWave;
  const S* src = static_cast<const S*>(w);
  if (nv <= 2) hipLaunchKernelGGL((quant_rows_e4m3_vec_kernel<El, 2>), grid, dim3(kThreads), 0, s, src, rows, cols, q, scales, row_ids, id_count, numel);
  else if (nv <= 4) hipLaunchKernelGGL((quant_rows_e4m3_vec_kernel<El, 4>), grid, dim3(kThreads), 0, s, src, rows, cols, q, scales, row_ids, id_count, numel);
  else hipLaunchKernelGGL((quant_rows_e4m3_vec_kernel<El, 8>), grid, dim3(kThreads), 0, s, src, rows, cols, q, scales, row_ids, id_count, numel);
  return true;
}

int grid_for(int64_t work_items) {
  int64_t b = (work_items + kThreads - 1) / kThreads;
  const int64_t cap = 256 * 16;  // 256 CUs, 16 workgroups each; the loops stride past this
  if (b > cap) b = cap;
  if (b < 1) b = 1;
  return static_cast<int>(b);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename El>
int launch_silu(void* out, const void* in, int64_t rows, int d, hipStream_t s) {
  using S = typename El::S;
  constexpr int V = 16 / sizeof(S);
  if (d % V == 0 && aligned16(out) && aligned16(in))
    hipLaunchKernelGGL((silu_and_mul_kernel<El, V>), dim3(grid_for(rows * (d / V))), dim3(kThreads),
                       0, s, static_cast<S*>(out), static_cast<const S*>(in), rows, d);
  else
    hipLaunchKernelGGL((silu_and_mul_kernel<El, 1>), dim3(grid_for(rows * d)), dim3(kThreads), 0, s,
                       static_cast<S*>(out), static_cast<const S*>(in), rows, d);
  return moe_check_launch("silu_and_mul");
}

template <typename El>
int launch_swiglu(void* out, const void* in, int64_t rows, int d, float alpha, float limit,
                  hipStream_t s) {
  using S = typename El::S;
  constexpr int V = 8 / sizeof(S);  // the input vector is twice as wide
  if (d % V == 0 && aligned16(in) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0)
    hipLaunchKernelGGL((swigluoai_and_mul_kernel<El, V>), dim3(grid_for(rows * (d / V))),
                       dim3(kThreads), 0, s, static_cast<S*>(out), static_cast<const S*>(in), rows,
                       d, alpha, limit);
  else
    hipLaunchKernelGGL((swigluoai_and_mul_kernel<El, 1>), dim3(grid_for(rows * d)), dim3(kThreads),
                       0, s, static_cast<S*>(out), static_cast<const S*>(in), rows, d, alpha, limit);
  return moe_check_launch("swigluoai_and_mul");
}

template <typename El>
int launch_sum(void* out, const void* in, int64_t T, int K, int H, hipStream_t s) {
  using S = typename El::S;
  constexpr int V = 16 / sizeof(S);
  if (H % V == 0 && aligned16(out) && aligned16(in))
    hipLaunchKernelGGL((moe_sum_kernel<El, V>), dim3(grid_for(T * (H / V))), dim3(kThreads), 0, s,
                       static_cast<S*>(out), static_cast<const S*>(in), T, K, H);
  else
    hipLaunchKernelGGL((moe_sum_kernel<El, 1>), dim3(grid_for(T * H)), dim3(kThreads), 0, s,
                       static_cast<S*>(out), static_cast<const S*>(in), T, K, H);
  return moe_check_launch("moe_sum");
}

}  // namespace

MOE_EXPORT int moe_silu_and_mul(void* out, const void* in, int64_t rows, int d, int dtype,
                                void* stream) {
  if (rows < 0 || d < 1) return moe_fail(MOE_ERR_ARG, "silu_and_mul: bad sizes rows=%lld d=%d", static_cast<long long>(rows), d);
  if (rows == 0) return MOE_OK;
  if (!out || !in) return moe_fail(MOE_ERR_ARG, "silu_and_mul: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MOE_F32: return launch_silu<ElemF32>(out, in, rows, d, s);
    case MOE_F16: return launch_silu<ElemF16>(out, in, rows, d, s);
    case MOE_BF16: return launch_silu<ElemBF16>(out, in, rows, d, s);
    default: return moe_fail(MOE_ERR_ARG, "silu_and_mul: unsupported dtype code %d", dtype);
  }
}

MOE_EXPORT int moe_swigluoai_and_mul(void* out, const void* in, int64_t rows, int d, int dtype,
                                     float alpha, float limit, void* stream) {
  if (rows < 0 || d < 1) return moe_fail(MOE_ERR_ARG, "swigluoai_and_mul: bad sizes rows=%lld d=%d", static_cast<long long>(rows), d);
  if (rows == 0) return MOE_OK;
  if (!out || !in) return moe_fail(MOE_ERR_ARG, "swigluoai_and_mul: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MOE_F32: return launch_swiglu<ElemF32>(out, in, rows, d, alpha, limit, s);
    case MOE_F16: return launch_swiglu<ElemF16>(out, in, rows, d, alpha, limit, s);
    case MOE_BF16: return launch_swiglu<ElemBF16>(out, in, rows, d, alpha, limit, s);
    default: return moe_fail(MOE_ERR_ARG, "swigluoai_and_mul: unsupported dtype code %d", dtype);
  }
}

MOE_EXPORT int moe_sum(void* out, const void* in, int64_t T, int K, int H, int dtype,
                       void* stream) {
  if (T < 0 || K < 1 || H < 1) return moe_fail(MOE_ERR_ARG, "moe_sum: bad sizes T=%lld K=%d H=%d", static_cast<long long>(T), K, H);
  if (T == 0) return MOE_OK;
  if (!out || !in) return moe_fail(MOE_ERR_ARG, "moe_sum: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MOE_F32: return launch_sum<ElemF32>(out, in, T, K, H, s);
    case MOE_F16: return launch_sum<ElemF16>(out, in, T, K, H, s);
    case MOE_BF16: return launch_sum<ElemBF16>(out, in, T, K, H, s);
    default: return moe_fail(MOE_ERR_ARG, "moe_sum: unsupported dtype code %d", dtype);
  }
}

MOE_EXPORT int moe_quant_rows_e4m3(const void* w, int src_dtype, int64_t rows, int cols,
                                   uint8_t* q, float* scales, void* stream) {
  return moe_quant_slot_rows_e4m3(w, src_dtype, rows, cols, q, scales, nullptr, 0, 0, stream);
}

// Row r is skipped (q and scales left untouched) when row_ids is given and r >= id_count or
// row_ids[r] >= numel: the padding slots of an expert-sorted intermediate.
int moe_quant_slot_rows_e4m3(const void* w, int src_dtype, int64_t rows, int cols, uint8_t* q,
                             float* scales, const int32_t* row_ids, int64_t id_count, int numel,
                             void* stream) {
  if (rows < 0 || cols < 1) return moe_fail(MOE_ERR_ARG, "quant_rows_e4m3: bad sizes rows=%lld cols=%d", static_cast<long long>(rows), cols);
  if (rows == 0) return MOE_OK;
  if (!w || !q || !scales) return moe_fail(MOE_ERR_ARG, "quant_rows_e4m3: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t blocks = (rows + kThreads / kWave - 1) / (kThreads / kWave);
  if (blocks > INT32_MAX) return moe_fail(MOE_ERR_ARG, "quant_rows_e4m3: too many rows");
  const dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
  switch (src_dtype) {
    case MOE_F32:
      hipLaunchKernelGGL(quant_rows_e4m3_kernel<ElemF32>, grid, block, 0, s, static_cast<const float*>(w), rows, cols, q, scales, row_ids, id_count, numel);
      break;
    case MOE_F16:
      if (!launch_quant_vec<ElemF16>(w, rows, cols, q, scales, row_ids, id_count, numel, grid, s))
        hipLaunchKernelGGL(quant_rows_e4m3_kernel<ElemF16>, grid, block, 0, s, static_cast<const uint16_t*>(w), rows, cols, q, scales, row_ids, id_count, numel);
      break;
    case MOE_BF16:
      if (!launch_quant_vec<ElemBF16>(w, rows, cols, q, scales, row_ids, id_count, numel, grid, s))
        hipLaunchKernelGGL(quant_rows_e4m3_kernel<ElemBF16>, grid, block, 0, s, static_cast<const uint16_t*>(w), rows, cols, q, scales, row_ids, id_count, numel);
      break;
    default:
      return moe_fail(MOE_ERR_ARG, "quant_rows_e4m3: unsupported source dtype code %d", src_dtype);
  }
  return moe_check_launch("quant_rows_e4m3");
}
