// Shared host/device helpers for libmoe_gfx950.so (gfx950 / CDNA4 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/moe_gfx950.h"

#define MOE_EXPORT extern "C" __attribute__((visibility("default")))

// Records a thread-local message and returns `code`.
int moe_fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Checks hipGetLastError() after a launch; 0 or MOE_ERR_LAUNCH.
int moe_check_launch(const char* what);

// moe_quant_rows_e4m3 restricted to the live slots of an expert-sorted matrix (library-internal).
int moe_quant_slot_rows_e4m3(const void* w, int src_dtype, int64_t rows, int cols, uint8_t* q,
                             float* scales, const int32_t* row_ids, int64_t id_count, int numel,
                             void* stream);

// Dynamic LDS above 64 KB must be opted into once per kernel and device.  One MoeLdsOptIn
// per kernel instantiation (a zero-initialised static); moe_opt_in_lds sets the attribute on
// the current device when it has not been set there yet.  Safe from several host threads.
constexpr int kMoeMaxDevices = 64;
struct MoeLdsOptIn {
  std::atomic<bool> done[kMoeMaxDevices];
};
int moe_opt_in_lds(MoeLdsOptIn& flags, const void* kernel, int lds_bytes, const char* what);

// int32 index, inside the 256-byte table of per-XCD ranges at the end of a moe_fused_experts
// workspace, of the count of expired waits of the one-launch form (cleared with the plan).
constexpr int kMoeStatusWord = 16;

static inline int64_t moe_align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// bf16 / f16 scalar conversions with explicit rounding (round to nearest even)
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  _Float16 v;
  __builtin_memcpy(&v, &h, 2);
  return static_cast<float>(v);
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 v = static_cast<_Float16>(f);  // v_cvt_f16_f32, round to nearest even
  uint16_t h;
  __builtin_memcpy(&h, &v, 2);
  return h;
}

// Element traits used by the elementwise kernels: storage type, load, store.
struct ElemF32 {
  using S = float;
  static __device__ __forceinline__ float ld(S v) { return v; }
  static __device__ __forceinline__ S st(float v) { return v; }
};
struct ElemBF16 {
  using S = uint16_t;
  static __device__ __forceinline__ float ld(S v) { return bf16_bits_to_f32(v); }
  static __device__ __forceinline__ S st(float v) { return f32_to_bf16_bits(v); }
};
struct ElemF16 {
  using S = uint16_t;
  static __device__ __forceinline__ float ld(S v) { return f16_bits_to_f32(v); }
  static __device__ __forceinline__ S st(float v) { return f32_to_f16_bits(v); }
};

// ---------------------------------------------------------------------------
// exp in fp32 as a fixed sequence of IEEE operations: Cody-Waite reduction by
// ln2 (two constants), degree-6 polynomial evaluated with fused multiply-adds,
// scaling through the exponent field.  <= 2 ulp.  Inputs above 88 give +inf,
// inputs below -104 give 0; between about -87.3 and -104 the result is
// subnormal, as CUDA's expf returns it when built without flush-to-zero (the
// reference's build, setup.py:46-47): such results are scaled in two steps, by
// 2^(n+64) through the exponent field (exact) and by one multiplication with
// 2^-64, which rounds once.  gfx950 code objects keep fp32 subnormals (denormal
// mode 3).  Translation units that use it are compiled with -ffp-contract=off
// so that no other operation is fused.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float moe_expf(float x) {
  if (x != x) return x;
  if (x > 88.0f) return __builtin_inff();
  if (x < -104.0f) return 0.0f;
  float n = __builtin_rintf(x * 1.44269504088896341f);
  float r = __builtin_fmaf(n, -0.693359375f, x);
  r = __builtin_fmaf(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = __builtin_fmaf(p, r, 1.3981999507e-3f);
  p = __builtin_fmaf(p, r, 8.3334519073e-3f);
  p = __builtin_fmaf(p, r, 4.1665795894e-2f);
  p = __builtin_fmaf(p, r, 1.6666665459e-1f);
  p = __builtin_fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  p = __builtin_fmaf(p, r2, r);
  p = p + 1.0f;
  int32_t ni = static_cast<int32_t>(n);
  if (ni < -125) {
    const float t = __uint_as_float(__float_as_uint(p) + (static_cast<uint32_t>(ni + 64) << 23));
    return t * 5.42101086242752217e-20f;  // 2^-64
  }
  return __uint_as_float(__float_as_uint(p) + (static_cast<uint32_t>(ni) << 23));
}

__device__ __forceinline__ float moe_silu(float x) { return x / (1.0f + moe_expf(-x)); }

__device__ __forceinline__ float moe_swigluoai(float g, float u, float alpha, float limit) {
  float cg = g > limit ? limit : g;
  float cu = u > limit ? limit : (u < -limit ? -limit : u);
  float sig = 1.0f / (1.0f + moe_expf(-cg * alpha));
  float glu = cg * sig;
  float r = (cu + 1.0f) * glu;
  // The product is an fp32 value before it is narrowed, as in the reference's kernel.  Without
  // this the compiler may fold the multiplication into the conversion to fp16 (one rounding
  // of the exact product instead of two), which differs in one element in ten thousand.
  asm volatile("" : "+v"(r));
  return r;
}
