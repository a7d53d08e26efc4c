/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement (scalar C, one thread) of the
 * integer / bit-level part of the fused-MoE expert path of
 * scale-snu/layered-prefill.  Nothing in the shipped library or the Python
 * package may link, load or call this file; only tests/, the smoke check and
 * the cpu_baseline leg of bench.py do, and only as the checker.
 *
 * What is restated, and from where (paths relative to the reference tree):
 *   oracle_topk_softmax          csrc/moe_topk_softmax_kernels.cu:182-380 (fused
 *                                power-of-two kernel), :50-166 (fallback),
 *                                :421-503 (dispatch); renormalisation from
 *                                nanovllm/layers/for_moe/fused_moe.py:417-418
 *   oracle_moe_align_block_size  csrc/moe_align_block_size_kernels.cu:140-291,
 *                                stable order from :92-110 and
 *                                nanovllm/layers/for_moe/fused_moe.py:42-55
 *   oracle_silu_and_mul_*        csrc/activation_kernels.cu:8-25,68-87
 *   oracle_swigluoai_and_mul_*   csrc/activation_kernels.cu:27-64,89-109
 *
 * Parity status
 *   - moe_align_block_size: pinned by the two worked examples in the
 *     reference's comments, by numpy stable argsort, and by brute force.
 *   - topk_softmax indices: pinned by closed form (softmax is monotone, so
 *     the ids equal a stable descending sort of the logits wherever the fp32
 *     probabilities are distinct) and brute force.
 *   - topk_softmax weights: the reference calls CUDA's expf, which is not in
 *     the reference tree (CUDA toolkit 12.8 libdevice).  This oracle defines
 *     its own fp32 exp (oracle_expf: Cody-Waite reduction + degree-6
 *     polynomial, every operation an IEEE fp32 operation or an fmaf), checked
 *     to <= 2 ulp against double-precision exp, subnormal results included:
 *     the reference is built without flush-to-zero (setup.py:46-47), so
 *     probabilities between 2^-149 and 2^-126 keep their value and their
 *     rank, as they do here.  The *bits* of the weights
 *     are therefore "parity unpinned" against the reference; their values
 *     agree with a float64 softmax to ~1e-7 relative.
 *   - The fallback path (E not a power of two, or E > 256) uses cub
 *     BlockReduce in the reference, whose summation order lives in the CUDA
 *     toolkit: the order used here (64 strided partial sums, then an xor
 *     butterfly) is this build's own -> weights' last bits "parity unpinned".
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; fmaf comes from libm,
 * so no -mfma / -march flag is needed and the .so runs on any x86-64 host).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* fp32 exp with a fully specified sequence of IEEE operations.        */
/* ------------------------------------------------------------------ */
static inline float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

ORACLE_API float oracle_expf(float x) {
  if (x != x) return x;
  if (x > 88.0f) return INFINITY;
  if (x < -104.0f) return 0.0f; /* below 2^-150: rounds to zero */
  float n = rintf(x * 1.44269504088896341f);
  float r = fmaf(n, -0.693359375f, x);         /* ln2 high part, 9 bits */
  r = fmaf(n, 2.12194440e-4f, r);              /* minus ln2 low part    */
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  p = fmaf(p, r2, r);
  p = p + 1.0f;
  /* scale by 2^n through the exponent field; p in [0.70, 1.42], n in
     [-150, 127] after the cut-offs above.  A result that may be subnormal
     (n <= -126) is scaled in two steps, p * 2^(n+64) through the field (exact)
     and one IEEE multiplication by 2^-64, which rounds once: the reference is
     built without flush-to-zero (setup.py:46-47, plain -O3), so CUDA's expf
     returns subnormals down to about -103.97 and so does this one. */
  int32_t ni = (int32_t)n;
  if (ni < -125) {
    float t = bits_to_float(float_to_bits(p) + ((uint32_t)(ni + 64) << 23));
    return t * 5.42101086242752217e-20f; /* 2^-64 */
  }
  return bits_to_float(float_to_bits(p) + ((uint32_t)ni << 23));
}

ORACLE_API void oracle_expf_array(const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = oracle_expf(x[i]);
}

/* ------------------------------------------------------------------ */
/* Router: softmax + iterative top-k                                   */
/* ------------------------------------------------------------------ */

/* Thread geometry of the fused kernel for a power-of-two expert count,
   csrc/moe_topk_softmax_kernels.cu:385-394,401-406. */
static void pow2_geometry(int E, int* elts_per_ldg, int* vpt, int* tpr) {
  int bytes = 16 < 4 * E ? 16 : 4 * E;
  int epl = bytes / 4;
  int vecs = E / (epl * 32);
  if (vecs < 1) vecs = 1;
  *elts_per_ldg = epl;
  *vpt = vecs * epl;
  *tpr = E / *vpt;
}

/* Column held in slot `ii` of thread `t` of a row group (:236-257,307-316). */
static inline int pow2_col(int t, int ii, int epl, int tpr) {
  return (ii / epl) * (epl * tpr) + t * epl + (ii % epl);
}

static void softmax_row_pow2(const float* x, float* p, int E) {
  int epl, vpt, tpr;
  pow2_geometry(E, &epl, &vpt, &tpr);
  float tmax[32], tsum[32];
  /* per-thread max in slot order, then xor butterfly (:261-273) */
  for (int t = 0; t < tpr; ++t) {
    float m = x[pow2_col(t, 0, epl, tpr)];
    for (int ii = 1; ii < vpt; ++ii) m = fmaxf(m, x[pow2_col(t, ii, epl, tpr)]);
    tmax[t] = m;
  }
  for (int mask = tpr / 2; mask > 0; mask /= 2) {
    float nxt[32];
    for (int t = 0; t < tpr; ++t) nxt[t] = fmaxf(tmax[t], tmax[t ^ mask]);
    memcpy(tmax, nxt, sizeof(float) * tpr);
  }
  /* exp and per-thread sum in slot order, then xor butterfly (:277-290) */
  for (int t = 0; t < tpr; ++t) {
    float s = 0.f;
    for (int ii = 0; ii < vpt; ++ii) {
      int c = pow2_col(t, ii, epl, tpr);
      p[c] = oracle_expf(x[c] - tmax[t]);
      s += p[c];
    }
    tsum[t] = s;
  }
  for (int mask = tpr / 2; mask > 0; mask /= 2) {
    float nxt[32];
    for (int t = 0; t < tpr; ++t) nxt[t] = tsum[t] + tsum[t ^ mask];
    memcpy(tsum, nxt, sizeof(float) * tpr);
  }
  /* scale by the reciprocal (:297-303) */
  float rinv = 1.f / tsum[0];
  for (int c = 0; c < E; ++c) p[c] = p[c] * rinv; /* subnormal products are kept (:297-303) */
}

/* Fallback for any other E (:50-106): 64 strided partial results combined by
   an xor butterfly 32,16,...,1. */
static void softmax_row_generic(const float* x, float* p, int E) {
  float part[64];
  for (int l = 0; l < 64; ++l) {
    float m = -INFINITY;
    for (int c = l; c < E; c += 64) m = fmaxf(m, x[c]);
    part[l] = m;
  }
  for (int mask = 32; mask > 0; mask /= 2) {
    float nxt[64];
    for (int l = 0; l < 64; ++l) nxt[l] = fmaxf(part[l], part[l ^ mask]);
    memcpy(part, nxt, sizeof(part));
  }
  float mx = part[0];
  for (int l = 0; l < 64; ++l) {
    float s = 0.f;
    for (int c = l; c < E; c += 64) {
      p[c] = oracle_expf(x[c] - mx);
      s += p[c];
    }
    part[l] = s;
  }
  for (int mask = 32; mask > 0; mask /= 2) {
    float nxt[64];
    for (int l = 0; l < 64; ++l) nxt[l] = part[l] + part[l ^ mask];
    memcpy(part, nxt, sizeof(part));
  }
  float rinv = 1.f / part[0];
  for (int c = 0; c < E; ++c) p[c] = p[c] * rinv;
}

/* Returns 0, or -1 on bad arguments.  `probs_or_null` (T*E floats) receives
   the softmax when given.  renormalize != 0 applies
   nanovllm/layers/for_moe/fused_moe.py:417-418 with the k-sum taken in
   ascending k. */
ORACLE_API int oracle_topk_softmax(const float* gating, float* topk_weights,
                                   int32_t* topk_ids,
                                   int32_t* token_expert_indices,
                                   float* probs_or_null, int T, int E, int K,
                                   int renormalize) {
  if (T < 0 || E <= 0 || K <= 0 || K > E) return -1;
  int pow2 = (E & (E - 1)) == 0 && E <= 256;
  float* p = (float*)malloc(sizeof(float) * (size_t)E);
  if (!p) return -1;
  for (int r = 0; r < T; ++r) {
    const float* x = gating + (size_t)r * E;
    if (pow2)
      softmax_row_pow2(x, p, E);
    else
      softmax_row_generic(x, p, E);
    if (probs_or_null) memcpy(probs_or_null + (size_t)r * E, p, sizeof(float) * E);
    for (int k = 0; k < K; ++k) {
      /* strict '>' in ascending column order == lowest index wins ties
         (:325, :343) */
      int best = 0;
      float bv = p[0];
      for (int c = 1; c < E; ++c)
        if (p[c] > bv) {
          bv = p[c];
          best = c;
        }
      topk_weights[(size_t)r * K + k] = bv;
      topk_ids[(size_t)r * K + k] = best;
      token_expert_indices[(size_t)r * K + k] = k * T + r; /* :362 */
      p[best] = -10000.f;                                  /* :376 */
    }
    if (renormalize) {
      float s = 0.f;
      for (int k = 0; k < K; ++k) s += topk_weights[(size_t)r * K + k];
      for (int k = 0; k < K; ++k)
        topk_weights[(size_t)r * K + k] = topk_weights[(size_t)r * K + k] / s;
    }
  }
  free(p);
  return 0;
}

/* ------------------------------------------------------------------ */
/* Expert-sorted token alignment                                       */
/* ------------------------------------------------------------------ */
enum { ID_I32 = 0, ID_I64 = 1, ID_I16 = 2, ID_I8 = 3, ID_U8 = 4 };

static inline int64_t load_id(const void* ids, int dtype, int64_t i) {
  switch (dtype) {
    case ID_I32: return ((const int32_t*)ids)[i];
    case ID_I64: return ((const int64_t*)ids)[i];
    case ID_I16: return ((const int16_t*)ids)[i];
    case ID_I8: return ((const int8_t*)ids)[i];
    default: return ((const uint8_t*)ids)[i];
  }
}

/* sorted_token_ids has capacity P = numel + E*(BM-1); expert_ids has capacity
   B = ceil(P/BM) (nanovllm/layers/for_moe/fused_moe.py:57-66).  Ids >= E are
   dropped (csrc/moe_align_block_size_kernels.cu:170-172,231-233); negative
   ids, which the reference would use as an out-of-bounds index, are dropped
   too.  Inside one expert's segment flat indices ascend (:92-110). */
ORACLE_API int oracle_moe_align_block_size(const void* topk_ids, int ids_dtype,
                                           int64_t numel, int E, int BM,
                                           int32_t* sorted_token_ids,
                                           int64_t sorted_cap,
                                           int32_t* expert_ids,
                                           int64_t expert_cap,
                                           int32_t* num_tokens_post_pad) {
  if (E <= 0 || BM <= 0 || numel < 0) return -1;
  int64_t* cnt = (int64_t*)calloc((size_t)E + 1, sizeof(int64_t));
  int64_t* cum = (int64_t*)calloc((size_t)E + 1, sizeof(int64_t));
  if (!cnt || !cum) return -1;
  for (int64_t i = 0; i < numel; ++i) {
    int64_t e = load_id(topk_ids, ids_dtype, i);
    if (e >= 0 && e < E) cnt[e]++;
  }
  for (int e = 0; e < E; ++e)
    cum[e + 1] = cum[e] + (cnt[e] + BM - 1) / BM * BM; /* :190-201 */
  int64_t total = cum[E];
  if (total > sorted_cap || (total + BM - 1) / BM > expert_cap) {
    free(cnt);
    free(cum);
    return -2;
  }
  for (int64_t i = 0; i < sorted_cap; ++i) sorted_token_ids[i] = (int32_t)numel; /* :150-152 */
  for (int e = 0; e < E; ++e)
    for (int64_t i = cum[e]; i < cum[e + 1]; i += BM) expert_ids[i / BM] = e; /* :205-210 */
  for (int64_t b = total / BM; b < expert_cap; ++b) expert_ids[b] = 0;        /* :212-217 */
  *num_tokens_post_pad = (int32_t)total;                                      /* :199-201 */
  int64_t* run = (int64_t*)calloc((size_t)E, sizeof(int64_t));
  if (!run) return -1;
  for (int64_t i = 0; i < numel; ++i) {
    int64_t e = load_id(topk_ids, ids_dtype, i);
    if (e < 0 || e >= E) continue;
    sorted_token_ids[cum[e] + run[e]++] = (int32_t)i;
  }
  free(run);
  free(cnt);
  free(cum);
  return 0;
}

/* ------------------------------------------------------------------ */
/* Gated activations                                                   */
/* ------------------------------------------------------------------ */
static inline float bf16_to_f32(uint16_t h) { return bits_to_float((uint32_t)h << 16); }
static inline uint16_t f32_to_bf16(float f) { /* round to nearest even */
  uint32_t u = float_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
ORACLE_API uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }

static inline float silu_f32(float x) { /* csrc/activation_kernels.cu:9-12 */
  return x / (1.0f + oracle_expf(-x));
}

/* out[r,i] = T(silu(in[r,i])) * in[r,d+i], the product taken in T
   (csrc/activation_kernels.cu:19-24). */
ORACLE_API void oracle_silu_and_mul_f32(float* out, const float* in, int64_t rows, int d) {
  for (int64_t r = 0; r < rows; ++r)
    for (int i = 0; i < d; ++i)
      out[r * d + i] = silu_f32(in[r * 2 * d + i]) * in[r * 2 * d + d + i];
}

ORACLE_API void oracle_silu_and_mul_bf16(uint16_t* out, const uint16_t* in, int64_t rows, int d) {
  for (int64_t r = 0; r < rows; ++r)
    for (int i = 0; i < d; ++i) {
      float x = bf16_to_f32(in[r * 2 * d + i]);
      float y = bf16_to_f32(in[r * 2 * d + d + i]);
      float s = bf16_to_f32(f32_to_bf16(silu_f32(x)));
      out[r * d + i] = f32_to_bf16(s * y); /* bf16*bf16 is exact in fp32 */
    }
}

/* swigluoai with interleaved gate/up (csrc/activation_kernels.cu:27-64):
   gate = in[r, 2i] clamped above by limit, up = in[r, 2i+1] clamped to
   [-limit, limit]; out = (up + 1) * gate * sigmoid(alpha * gate). */
static inline float swigluoai_f32(float g, float u, float alpha, float limit) {
  float cg = g > limit ? limit : g;
  float cu = u > limit ? limit : (u < -limit ? -limit : u);
  float sig = 1.0f / (1.0f + oracle_expf(-cg * alpha));
  float glu = cg * sig;
  return (cu + 1.0f) * glu;
}
ORACLE_API void oracle_swigluoai_and_mul_f32(float* out, const float* in, int64_t rows, int d,
                                             float alpha, float limit) {
  for (int64_t r = 0; r < rows; ++r)
    for (int i = 0; i < d; ++i)
      out[r * d + i] = swigluoai_f32(in[r * 2 * d + 2 * i], in[r * 2 * d + 2 * i + 1], alpha, limit);
}
ORACLE_API void oracle_swigluoai_and_mul_bf16(uint16_t* out, const uint16_t* in, int64_t rows,
                                              int d, float alpha, float limit) {
  for (int64_t r = 0; r < rows; ++r)
    for (int i = 0; i < d; ++i)
      out[r * d + i] = f32_to_bf16(swigluoai_f32(bf16_to_f32(in[r * 2 * d + 2 * i]),
                                                 bf16_to_f32(in[r * 2 * d + 2 * i + 1]), alpha,
                                                 limit));
}
