// Grouped expert GEMMs on CDNA4 matrix cores (bf16 / fp16 inputs, fp32 accumulate).
//
// Replaces the Triton fused_moe_kernel of the reference
// (nanovllm/layers/for_moe/fused_moe.py:84-223) and the two element-wise passes
// around it (silu_and_mul at :598-603, the routed-weight multiply at :210-214):
//
//   pass 1  inter[pos, :]  = act( x[tok / top_k, :] . W13[e]^T )      (gated epilogue)
//   pass 2  c3[tok, :]     = ( inter[pos, :] . W2[e]^T ) * topk_weight[tok]
//
// `pos` is a slot of sorted_token_ids, `tok` the flat (token, k) index stored
// there, `e` = expert_ids[pos / block_size].  One workgroup (4 wavefronts)
// owns one block of BM slots and one strip of weight rows; both operands are
// K-contiguous, are staged through LDS in 64-wide K tiles (16-byte chunks,
// XOR-swizzled so that the 16 lanes of one LDS pass hit 16 distinct bank
// groups) and feed v_mfma_f32_32x32x16.  The weight fragment is the A operand
// and the token fragment the B operand, so that a lane ends up with four
// consecutive output columns of one token and stores them as one 8-byte word.
#include <stdlib.h>

#include "common.h"


namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

struct MmaBF16 {
  using El = ElemBF16;
  static constexpr int kEs = 2;  // bytes per input element
  static constexpr int kBigChunks = 1;  // large-tile kernel: 16-byte chunks per lane and MFMA step
  static __device__ __forceinline__ f32x16 mma(const uint4& a, const uint4& b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mma_big(const uint4 (&a)[1], const uint4 (&b)[1], f32x16 c) {
    return mma(a[0], b[0], c);
  }
};
struct MmaF16 {
  using El = ElemF16;
  static constexpr int kEs = 2;
  static constexpr int kBigChunks = 1;
  static __device__ __forceinline__ f32x16 mma(const uint4& a, const uint4& b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mma_big(const uint4 (&a)[1], const uint4 (&b)[1], f32x16 c) {
    return mma(a[0], b[0], c);
  }
};

// fp32 inputs through v_mfma_f32_32x32x2_f32: a 16-byte chunk holds four K
// elements, one per MFMA step (K = 2 per step: one element from each lane half).
struct MmaF32 {
  using El = ElemF32;
  static constexpr int kEs = 4;
  static __device__ __forceinline__ f32x16 mma(const uint4& a, const uint4& b, f32x16 c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
};

// e4m3 (OCP) inputs, one byte per element: a 16-byte chunk holds 16 K elements,
// i.e. the per-lane operands of two v_mfma_f32_32x32x16_fp8_fp8 steps.  OutEl is
// the dtype results are rounded to and stored in.
template <typename OutEl>
struct MmaE4M3 {
  using El = OutEl;
  static constexpr int kEs = 1;
  static __device__ __forceinline__ f32x16 mma(const uint4& a, const uint4& b, f32x16 c) {
    const long a0 = static_cast<long>(a.x) | (static_cast<long>(a.y) << 32);
    const long a1 = static_cast<long>(a.z) | (static_cast<long>(a.w) << 32);
    const long b0 = static_cast<long>(b.x) | (static_cast<long>(b.y) << 32);
    const long b1 = static_cast<long>(b.z) | (static_cast<long>(b.w) << 32);
    c = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a0, b0, c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a1, b1, c, 0, 0, 0);
  }
};

// e4m3 in the large-tile kernel: v_mfma_f32_32x32x64_f8f6f4 takes 32 bytes per
// lane and operand (K = 64 per step, elements 32 * (lane / 32) .. + 31 of the
// lane's row) and runs at twice the rate of the 16-bit and the older fp8
// instructions.  The block scales are fixed at 2^0 (E8M0 127).
typedef __attribute__((ext_vector_type(8))) int i32x8;
template <typename OutEl>
struct MmaE4M3Big {
  using El = OutEl;
  static constexpr int kEs = 1;
  static constexpr int kBigChunks = 2;
  static __device__ __forceinline__ f32x16 mma_big(const uint4 (&a)[2], const uint4 (&b)[2], f32x16 c) {
    const i32x8 av = {static_cast<int>(a[0].x), static_cast<int>(a[0].y), static_cast<int>(a[0].z), static_cast<int>(a[0].w),
                      static_cast<int>(a[1].x), static_cast<int>(a[1].y), static_cast<int>(a[1].z), static_cast<int>(a[1].w)};
    const i32x8 bv = {static_cast<int>(b[0].x), static_cast<int>(b[0].y), static_cast<int>(b[0].z), static_cast<int>(b[0].w),
                      static_cast<int>(b[1].x), static_cast<int>(b[1].y), static_cast<int>(b[1].z), static_cast<int>(b[1].w)};
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, 0, 0, 0, 127, 0, 127);
  }
};

struct GemmParams {
  const void* a;        // pass 1: x [T, lda]; pass 2: inter [sorted_cap, lda]
  const void* w;        // [E, rows, Kd], K contiguous
  void* c;              // pass 1: inter [sorted_cap, ldc]; pass 2: c3 [T*K, ldc]
  const void* bias;     // [E, rows] in the activation dtype, or null
  const float* topk_w;  // [T*K]
  const float* a_scale; // fp8 only: per-row scale of the A operand (indexed like the A rows)
  const float* w_scale; // fp8 only: per-weight-row scale, [E, rows]
  int64_t w_scale_stride_e;
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  int64_t w_stride_e, w_stride_n, bias_stride_e;
  int64_t lda, ldc;
  int Kd;            // reduction length
  int N;             // output columns per row (I for pass 1, H for pass 2)
  int numel;         // T * top_k
  int top_k;
  int num_m_blocks;  // ceil(sorted_cap / BM)
  int num_n_tiles;
  int a_by_slot;     // A row = slot (pass 2) instead of tok / top_k (pass 1)
  int mul_weight;    // multiply by topk_w[tok] in the epilogue
  int activation;    // MoeActivation (gated pass only)
  int interleaved;   // gate/up rows interleaved (2n, 2n+1) instead of halves (n, N+n)
  float alpha, limit;
  int64_t sorted_cap; // capacity of sorted_ids
  int align_bs;      // block size the alignment was made with (a multiple of the kernel's M tile)
  int m_major;       // workgroup order inside an XCD: all n-tiles of an m-block are neighbours
  const int32_t* xcd_bounds;  // large-tile kernel: m-block range [b[x], b[x+1]) of XCD x, or null
  int wt_stores;     // large-tile flush: results go out as device-scope write-through stores (one-launch hand-off)
  // Operands stored as 32 KB units, one per (256 rows, K tile of 128 bytes), each unit the exact
  // image it has in LDS (row r at r * 128, 16-byte chunk c of the row at chunk c ^ ((r >> 1) & 7)):
  int w_tiled;       // weights: units [expert][n-tile][K tile] (moe_tile_expert_weights)
  int a_tiled;       // A operand of the down pass: units [m-block][K tile]
  int c_tiled;       // result of the gate-up pass written as such units
  int ragged;        // rows are not whole 16-byte chunks (K or a stride not a multiple of 16 bytes, or a
                     // base that is not 16-byte aligned): the register-staged kernel loads element by element
};

constexpr int kThreads = 256;
constexpr int kBK = 64;                  // K elements per LDS tile
constexpr int kRowBytes = kBK * 2;       // 128 B per staged row
constexpr int kXcds = 8;

__device__ __forceinline__ int swizzled(int row, int chunk) {
  return row * kRowBytes + ((chunk ^ ((row >> 1) & 7)) << 4);
}


// Writes one 32x32 accumulator fragment (pair, when gated): this lane holds, for
// token `tok` (slot `slot`), the output columns ncol0 + 8*g + i, g,i in 0..3.
// `rw` is the routed weight of the slot when the pass applies it, else 1.
// Rounding follows the reference's storage points: the GEMM result is rounded to
// the activation dtype, silu is rounded, the product is rounded
// (nanovllm/layers/for_moe/fused_moe.py:216, csrc/activation_kernels.cu:11,23).
template <typename El, bool GATED>
__device__ __forceinline__ void store_fragment(const GemmParams& p, int e, const f32x16& ga,
                                               const f32x16& ua, int tok, int slot, int ncol0, float rw) {
  using S = typename El::S;
  const S* bias = static_cast<const S*>(p.bias);
  // fp8: the accumulator is in units of (activation scale x weight scale)
  const float as = p.a_scale ? p.a_scale[p.a_by_slot ? slot : tok / p.top_k] : 1.f;
  const float* ws = p.w_scale ? p.w_scale + e * p.w_scale_stride_e : nullptr;
  const int64_t crow = p.a_by_slot ? tok : slot;  // pass 2 writes by token, pass 1 by slot
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int n = ncol0 + 8 * g;
    S o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = (n + i < p.N) ? n + i : p.N - 1;
      if constexpr (GATED) {
        float gv = ga[4 * g + i], uv = ua[4 * g + i];
        if (ws) {
          gv *= as * ws[p.interleaved ? 2 * col : col];
          uv *= as * ws[p.interleaved ? 2 * col + 1 : p.N + col];
        }
        if (bias) {
          const int64_t grow = p.interleaved ? 2 * col : col;
          const int64_t urow = p.interleaved ? 2 * col + 1 : p.N + col;
          gv += El::ld(bias[e * p.bias_stride_e + grow]);
          uv += El::ld(bias[e * p.bias_stride_e + urow]);
        }
        if (p.mul_weight) { gv *= rw; uv *= rw; }
        gv = El::ld(El::st(gv));
        uv = El::ld(El::st(uv));
        float r;
        if (p.activation == MOE_ACT_SILU) {
          r = El::ld(El::st(moe_silu(gv))) * uv;
        } else if (p.activation == MOE_ACT_SWIGLUOAI) {
          r = moe_swigluoai(gv, uv, p.alpha, p.limit);
        } else {
          const float ge = 0.5f * gv * (1.f + erff(gv * 0.70710678118654752f));
          r = El::ld(El::st(ge)) * uv;
        }
        o[i] = El::st(r);
      } else {
        float v = ga[4 * g + i];
        if (ws) v *= as * ws[col];
        if (bias) v += El::ld(bias[e * p.bias_stride_e + col]);
        o[i] = El::st(v * rw);
      }
    }
    S* dst = static_cast<S*>(p.c) + crow * p.ldc + n;
    if (n + 3 < p.N && (p.ldc & 3) == 0) {
      if constexpr (sizeof(S) == 4) {
        *reinterpret_cast<float4*>(dst) = float4{o[0], o[1], o[2], o[3]};
      } else {
        *reinterpret_cast<uint2*>(dst) = uint2{static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16),
                                               static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16)};
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < p.N) dst[i] = o[i];
    }
  }
}

// One 16-byte chunk of a row whose start is only element-aligned and of which only the first
// `valid` elements exist (the rest reads as zero): what the Triton kernel of the reference does with
// its K mask (nanovllm/layers/for_moe/fused_moe.py:191-205,218-223).
template <int ES>
__device__ __forceinline__ uint4 load_chunk_by_element(const char* ptr, int valid) {
  uint32_t w[4] = {0, 0, 0, 0};
  if constexpr (ES == 4) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < valid) w[i] = reinterpret_cast<const uint32_t*>(ptr)[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < valid) w[i >> 1] |= static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(ptr)[i]) << (16 * (i & 1));
  }
  return uint4{w[0], w[1], w[2], w[3]};
}

// RAGGED: operand rows are read element by element with a mask on K (any H, I, stride and
// element-aligned base); the results are those of the 16-byte path wherever both apply.
template <typename Mma, int BM, int BNW, int WAVES_M, bool GATED, bool RAGGED = false>
__global__ __launch_bounds__(kThreads) void grouped_gemm_kernel(const GemmParams p) {
  using El = typename Mma::El;
  constexpr int ES = Mma::kEs;               // bytes per input element
  constexpr int BKE = kRowBytes / ES;        // K elements per staged 128-byte row
  constexpr int CE = 16 / ES;                // K elements per 16-byte chunk
  constexpr int WAVES_N = 4 / WAVES_M;
  constexpr int TM = BM / WAVES_M, FM = TM / 32;     // token fragments per wavefront
  constexpr int TNW = BNW / WAVES_N, FN = TNW / 32;  // weight-row fragments per wavefront
  constexpr int FNO = GATED ? FN / 2 : FN;           // output fragments per wavefront
  constexpr int BN_OUT = GATED ? BNW / 2 : BNW;      // output columns per workgroup
  constexpr int A_LD = BM / 32, B_LD = BNW / 32;     // 16-byte chunks per thread and stage
  constexpr int STAGE_BYTES = (BM + BNW) * kRowBytes;
  static_assert(FM >= 1 && FNO >= 1, "tile too small for the wavefront layout");
  extern __shared__ __attribute__((aligned(16))) char smem[];

  // Workgroups are handed to the 8 XCDs round-robin; give each XCD one
  // contiguous range of the (n-tile major, m-block minor) order so that a strip
  // of expert weights is pulled through one L2 only.
  // The grid covers the worst-case padding; only the m-blocks below the padded
  // total are live, and the ranges are cut from those so every XCD gets the same share.
  const int live_mb = (*p.num_post_pad + BM - 1) / BM;
  const int live = live_mb * p.num_n_tiles;
  const int per_xcd = (live + kXcds - 1) / kXcds;
  const int xslot = blockIdx.x / kXcds;
  const int logical = (blockIdx.x % kXcds) * per_xcd + xslot;
  if (xslot >= per_xcd || logical >= live) return;
  int nt, mb;
  if (p.m_major) {
    mb = logical / p.num_n_tiles;
    nt = logical - mb * p.num_n_tiles;
  } else {
    nt = logical / live_mb;
    mb = logical - nt * live_mb;
  }
  // real slots come first in an alignment block: a tile that starts on padding is empty
  if (p.sorted_ids[mb * BM] >= p.numel) return;
  const int e = p.expert_ids[(mb * BM) / p.align_bs];
  const int n0 = nt * BN_OUT;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  const int ld_row = tid >> 3, ld_c = tid & 7;

  const char* a_src[A_LD];
#pragma unroll
  for (int j = 0; j < A_LD; ++j) {
    const int slot = mb * BM + ld_row + 32 * j;
    int64_t src = slot;
    if (!p.a_by_slot) {
      const int tok = p.sorted_ids[slot];
      src = tok < p.numel ? tok / p.top_k : 0;
    }
    a_src[j] = static_cast<const char*>(p.a) + (src * p.lda + ld_c * CE) * ES;
  }
  const char* w_src[B_LD];
#pragma unroll
  for (int j = 0; j < B_LD; ++j) {
    const int rr = ld_row + 32 * j;
    int64_t wrow;
    if constexpr (GATED) {
      const int half = rr / (BNW / 2);
      int n = n0 + rr % (BNW / 2);
      n = n < p.N ? n : p.N - 1;
      wrow = p.interleaved ? (2 * n + half) : (half * p.N + n);
    } else {
      const int n = n0 + rr;
      wrow = n < p.N ? n : p.N - 1;
    }
    w_src[j] = static_cast<const char*>(p.w) +
               (static_cast<int64_t>(e) * p.w_stride_e + wrow * p.w_stride_n + ld_c * CE) * ES;
  }
  const int st_off = swizzled(ld_row, ld_c);  // rows 32 apart share the swizzle

  // fragment read offsets
  const int l32 = lane & 31, lhi = lane >> 5;
  int rd_k[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) rd_k[kk] = ((2 * kk + lhi) ^ ((l32 >> 1) & 7)) << 4;
  int x_row[FM], w_row[FN];
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) x_row[fm] = (wm * TM + fm * 32 + l32) * kRowBytes;
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    int r;
    if constexpr (GATED)
      r = (fn < FNO) ? wn * (TNW / 2) + fn * 32 : BNW / 2 + wn * (TNW / 2) + (fn - FNO) * 32;
    else
      r = wn * TNW + fn * 32;
    w_row[fn] = (BM + r + l32) * kRowBytes;
  }

  f32x16 acc[FN][FM];
#pragma unroll
  for (int fn = 0; fn < FN; ++fn)
#pragma unroll
    for (int fm = 0; fm < FM; ++fm)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[fn][fm][r] = 0.f;

  uint4 a_reg[A_LD], b_reg[B_LD];
  const int nk = (p.Kd + BKE - 1) / BKE;

  auto gload = [&](int kt) {
    if constexpr (RAGGED) {
      static_assert(ES != 1, "e4m3 rows are whole 16-byte chunks");
      const int valid = p.Kd - (kt * BKE + ld_c * CE);
#pragma unroll
      for (int j = 0; j < A_LD; ++j) a_reg[j] = load_chunk_by_element<ES>(a_src[j] + kt * kRowBytes, valid);
#pragma unroll
      for (int j = 0; j < B_LD; ++j) b_reg[j] = load_chunk_by_element<ES>(w_src[j] + kt * kRowBytes, valid);
      return;
    }
    const bool in_k = kt * BKE + ld_c * CE < p.Kd;
#pragma unroll
    for (int j = 0; j < A_LD; ++j)
      a_reg[j] = in_k ? *reinterpret_cast<const uint4*>(a_src[j] + kt * kRowBytes) : uint4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < B_LD; ++j)
      b_reg[j] = in_k ? *reinterpret_cast<const uint4*>(w_src[j] + kt * kRowBytes) : uint4{0, 0, 0, 0};
  };
  auto sstore = [&](int stage) {
    char* base = smem + stage * STAGE_BYTES + st_off;
#pragma unroll
    for (int j = 0; j < A_LD; ++j) *reinterpret_cast<uint4*>(base + j * 32 * kRowBytes) = a_reg[j];
#pragma unroll
    for (int j = 0; j < B_LD; ++j)
      *reinterpret_cast<uint4*>(base + (BM + j * 32) * kRowBytes) = b_reg[j];
  };

  gload(0);
  sstore(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) gload(kt + 1);
    const char* st = smem + cur * STAGE_BYTES;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      uint4 xf[FM], wf[FN];
#pragma unroll
      for (int fm = 0; fm < FM; ++fm) xf[fm] = *reinterpret_cast<const uint4*>(st + x_row[fm] + rd_k[kk]);
#pragma unroll
      for (int fn = 0; fn < FN; ++fn) wf[fn] = *reinterpret_cast<const uint4*>(st + w_row[fn] + rd_k[kk]);
#pragma unroll
      for (int fn = 0; fn < FN; ++fn)
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) acc[fn][fm] = Mma::mma(wf[fn], xf[fm], acc[fn][fm]);
    }
    if (kt + 1 < nk) sstore(cur ^ 1);
    __syncthreads();
  }

  // Epilogue.  acc[fn][fm][r]: weight row 8*(r/4) + 4*(lane/32) + r%4 of
  // fragment fn, token row lane%32 of fragment fm.
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    const int slot = mb * BM + wm * TM + fm * 32 + l32;
    const int tok = p.sorted_ids[slot];
    if (tok >= p.numel) continue;  // padding slot
    const float rw = p.mul_weight ? p.topk_w[tok] : 1.f;
#pragma unroll
    for (int fo = 0; fo < FNO; ++fo) {
      const int ncol0 = n0 + (GATED ? wn * (TNW / 2) : wn * TNW) + fo * 32 + 4 * lhi;
      store_fragment<El, GATED>(p, e, acc[fo][fm], acc[GATED ? fo + FNO : fo][fm], tok, slot, ncol0, rw);
    }
  }
}


// ---------------------------------------------------------------------------
// Large-tile variant for compute-bound calls: 256 slots x 256 weight rows per
// workgroup, one wavefront per SIMD, each owning a 128 x 128 register tile
// (16 accumulator fragments in AGPRs), so one 16-byte fragment read from LDS
// feeds four MFMAs.  The vector-memory path delivers 64 B/clk per CU against
// 4096 MFMA flop/clk, so a tile needs >= 64 flop per loaded byte: 256 x 256
// gives 128, and rows are staged 128 bytes (64 K elements) at a time because
// a load that takes only half of a 128-byte line runs at half that rate.
// K advances in 64-element tiles.  A tile is two 32 KB units, its 256 token
// rows and its 256 weight rows, and LDS is a ring of five such units filled by
// direct global->LDS loads (global_load_lds_dwordx4, issued from inline assembly
// so that no compiler-inserted wait serialises them).  While tile kt is being
// multiplied, the weight unit of tile kt+1..kt+2 and the token unit of tile
// kt+2..kt+3 are in flight (up to 96 KB per CU: the loop is bound by how many
// bytes the CU keeps in flight towards L2, not by MFMA issue), and the only
// per-tile synchronisation is one wait plus one s_barrier.  16-byte chunk c of
// row r sits at chunk c ^ ((r >> 1) & 7), which makes both the DMA writes (8
// lanes per row) and the fragment reads (16 consecutive rows, one chunk) touch
// 16 distinct 16-byte
// bank groups.  Token fragments holding only padding slots are skipped and
// their rows are not loaded.
// The epilogue rounds the accumulators to the activation dtype, parks the
// wavefront's 128 x 128 tile in LDS and writes it out with 16-byte stores, the
// gated activation being applied on the way.
// ---------------------------------------------------------------------------
constexpr int kBigBM = 256, kBigBNW = 256, kBigBK = 64, kBigUnits = 5;
constexpr int kBigRowBytes = kBigBK * 2;
constexpr int kBigUnitBytes = 256 * kBigRowBytes;  // 256 rows of one operand, one K tile
constexpr int kBigDmaPerUnit = 8;                  // global_load_lds instructions per thread and unit
constexpr int kEpiRowBytes = 128 * 2 + 16;   // one token row of a wavefront's tile, padded
constexpr int kEpiWaveBytes = 128 * kEpiRowBytes;
constexpr int kBigLdsBytes = 4 * kEpiWaveBytes;    // epilogue staging, reuses the ring
constexpr int kBigSideBytes = 5 * kBigBM * 4;      // per slot: token id, routed weight, fp8 row scale; per weight row: fp8 scale, bias
constexpr int kBigLdsTotal = kBigUnits * kBigUnitBytes;  // the whole 160 KB of the CU
static_assert(kBigLdsBytes + kBigSideBytes + 32 <= kBigLdsTotal, "epilogue staging must fit in the ring");
constexpr int kBigStatusWord = kMoeStatusWord;

typedef __attribute__((address_space(3))) char lds_char;

__device__ __forceinline__ uint32_t lds_offset_of(const char* p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const lds_char*)p));
}

// 16 bytes per lane from global memory straight into LDS at
// lds_wave_base + 16 * lane.  `base` and `lds_wave_base` are wavefront-uniform.
__device__ __forceinline__ void lds_dma16(const char* base, uint32_t lane_byte_offset,
                                          uint32_t lds_wave_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(lds_wave_base), "v"(lane_byte_offset), "s"(base)
      : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void bare_barrier() {
  asm volatile("s_barrier" ::: "memory");
}

// 16-byte store that is written through to memory at device scope (sc1): once vmcnt has
// counted it, every XCD sees the data, with no write-back of the L2 needed.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
__device__ __forceinline__ void store16_device_scope(void* p, const uint4& v) {
  const u32x4 d = {v.x, v.y, v.z, v.w};
  asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(d) : "memory");
}

// x * sigmoid(x) with the hardware exp2 and reciprocal (about 1e-6 relative
// error); the result is rounded to 16 bits right after, so it differs from the
// exact-sequence moe_silu in well under one rounding in a thousand.
__device__ __forceinline__ float silu_fast(float x) {
  const float e = __builtin_amdgcn_exp2f(x * -1.44269504088896341f);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

template <typename El>
__device__ __forceinline__ uint32_t pack2(float a, float b);
template <>
__device__ __forceinline__ uint32_t pack2<ElemBF16>(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
template <>
__device__ __forceinline__ uint32_t pack2<ElemF16>(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, f16x2));
}

struct BigCtx {
  const char* a_base;   // wave-uniform base of the A rows
  const char* w_base;   // wave-uniform base of this expert's weights
  uint32_t a_off[8];    // per-lane byte offsets of the wavefront's eight requests of a unit (dma_win_bias included)
  uint32_t w_off[8];
  uint32_t dma_lds;     // LDS address of the middle of this wavefront's 8 KB DMA window in unit slot 0
  uint32_t dma_lds_light_a;  // the same for the 2 KB window of the first 64-row token unit of a weight-streaming tile
  int rd_k[4];          // fragment read offsets for the four MFMA steps of a K tile
  int x_row;            // byte offset of this wavefront's first token row in a token unit
  int w_row[4];         // byte offsets of this wavefront's weight fragments in a weight unit
  int a_step, w_step;   // bytes from one K tile to the next: 128 along a row, 32768 from unit to unit
};

template <int V>
struct IntTag { static constexpr int value = V; };

template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(IntTag<B>{});
    static_for<B + 1, E>(f);
  }
}

// 16 bytes per lane from global memory into LDS, the instruction's offset field added on both
// sides: the data of base + lane_byte_offset + OFF lands at M0 + OFF + 16 * lane.  A wavefront fills
// one contiguous window of a unit (8 KB of a 32 KB unit) with requests that differ in OFF only, so
// M0 is written once per window (SET_M0, on the first request; the s_nop is the wait state M0
// needs) instead of once per request: three scalar writes and wait states per K tile where there
// were sixteen (0.5 to 1 % of the launch at 8448 and at 256 tokens, results unchanged bit for bit).
// M0 has to keep its value from one request of a window to the next; nothing else in the K loops
// writes it (they are MFMAs, LDS reads, waits and these requests).
template <int OFF, bool SET_M0>
__device__ __forceinline__ void lds_dma16_rel(const char* base, uint32_t lane_byte_offset, uint32_t lds_m0) {
  static_assert(OFF >= -4096 && OFF <= 4095, "13-bit signed offset field");
  if constexpr (SET_M0) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %2 offset:%3"
        :
        : "s"(lds_m0), "v"(lane_byte_offset), "s"(base), "n"(OFF)
        : "memory");
  } else {
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(lane_byte_offset), "s"(base), "n"(OFF) : "memory");
  }
}
// Request J (0..7) of a wavefront's 8 KB window of a 32 KB unit; lds_mid = LDS address of the
// window's middle.  Unit byte 8192 * wave + 1024 * J + 16 * lane, i.e. row 64 * wave + 8 * J +
// lane / 8 of the unit, position lane % 8 of that row.
template <int J, bool SET_M0>
__device__ __forceinline__ void lds_dma16_win(const char* base, uint32_t lane_byte_offset, uint32_t lds_mid) {
  lds_dma16_rel<(J - 4) * 1024, SET_M0>(base, lane_byte_offset, lds_mid);
}
// What a per-lane offset of request J carries besides the data's offset from the operand's start:
// the offset field's share taken out again, and 4096 that the base pointers are short of (so that
// no offset is negative).
constexpr uint32_t dma_win_bias(int j) { return static_cast<uint32_t>(4096 - (j - 4) * 1024); }

// Main loop for a wavefront that has FMC live token fragments (0..4).
// Unit j of the stream  A(0) W(0) A(1) W(1) ...  lives in ring slot j % 5.
// The caller has requested W(0) and the first half of W(1) (when nk > 1) before
// anything else.  One K tile (128 bytes per row) is STEPS MFMA steps of CH 16-byte
// chunks per lane and operand: four steps of one chunk for the 16-bit dtypes, two
// steps of two chunks for e4m3.  Two register sets of fragments (P, Q) alternate,
// and every step carries, between its MFMAs, the LDS reads of the next step's
// fragments and its share of the sixteen DMA requests of the K tile:
//   steps 0 .. STEPS-2 of tile kt request W(kt+1)[4..7] and A(kt+2)[0..7]
//   wait for tile kt+1, barrier (frees the two slots of tile kt)
//   step STEPS-1 reads P(kt+1,0) and requests W(kt+2)[0..3]
// At the wait only A(kt+2), the youngest request, may still be outstanding.
// sched_barrier pins this order against the compiler's scheduler.
// The loop is bound by instruction issue (one wavefront per SIMD issues one
// instruction every four clocks, an MFMA takes 32), so a K tile is straight-line
// code: the two tiles at the end of K, which request less, are separate
// instances of the tile body instead of tests around every request, an LDS read
// is one instruction (lane base + slot in one addition per operand and step,
// everything else in the offset field), a DMA request three.
template <typename Mma, int FMC, bool GATED>
__device__ __forceinline__ void big_mainloop(const BigCtx& c, const char* smem, int nk,
                                             f32x16 (&acc)[4][4]) {
  constexpr int CH = Mma::kBigChunks, STEPS = 4 / CH;
  constexpr int PER = 12 / (STEPS - 1);  // requests carried by each of the first STEPS-1 steps
  constexpr int XF = FMC > 0 ? FMC : 1;
  constexpr int NM = 4 * FMC;            // MFMAs of a step
  // byte offset of weight fragment fn from fragment 0 inside a weight unit
  auto woff = [](int fn) { return GATED ? (fn < 2 ? fn * 4096 : 16384 + (fn - 2) * 4096) : fn * 4096; };
  // per-lane parts of the fragment addresses: chunk q of the K tile, token rows / weight rows
  int xl[4], wl[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    xl[q] = c.x_row + c.rd_k[q];
    wl[q] = c.w_row[0] + c.rd_k[q];
  }
  uint4 wfP[4][CH], xfP[XF][CH], wfQ[4][CH], xfQ[XF][CH];

  // One MFMA step on fragment set X.  Between its MFMAs: the LDS reads of set Y (chunks of
  // MFMA step YKK of the tile whose units start at byte ya / yw of the ring) when LOAD, and
  // requests [0, ND) of `dma`.  Spread out, because a burst of requests stalls the wavefront,
  // and with it the matrix pipe, until the queue drains.  Reads go out in the order the next
  // step consumes them: x0, w0..w3, x1, x2, x3.
  auto step = [&](auto nd_tag, auto load_tag, auto ykk_tag, const uint4 (&wfX)[4][CH], const uint4 (&xfX)[XF][CH],
                  uint4 (&wfY)[4][CH], uint4 (&xfY)[XF][CH], int ya, int yw, auto&& dma) {
    constexpr int ND = decltype(nd_tag)::value;
    constexpr bool LOAD = decltype(load_tag)::value != 0 && FMC > 0;
    constexpr int YKK = decltype(ykk_tag)::value;
    auto read_y = [&](auto rt) {
      constexpr int r = decltype(rt)::value;
      if constexpr (LOAD) {
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
          const char* sta = smem + (ya + xl[YKK * CH + ch]);
          const char* stw = smem + (yw + wl[YKK * CH + ch]);
          if constexpr (r == 0) xfY[0][ch] = *reinterpret_cast<const uint4*>(sta);
          else if constexpr (r <= 4) wfY[r - 1][ch] = *reinterpret_cast<const uint4*>(stw + woff(r - 1));
          else if constexpr (r - 4 < FMC) xfY[r - 4][ch] = *reinterpret_cast<const uint4*>(sta + (r - 4) * 4096);
        }
      }
    };
    static_for<0, (NM > 0 ? NM : 1)>([&](auto mt) {
      constexpr int m = decltype(mt)::value;
      if constexpr (NM > 0) acc[m & 3][m >> 2] = Mma::mma_big(wfX[m & 3], xfX[m >> 2], acc[m & 3][m >> 2]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr ((m & 1) == 0) read_y(IntTag<(m >> 1)>{});
      static_for<(m * ND) / 16, ((m + 1) * ND) / 16>([&](auto jt) { dma(jt); });
      __builtin_amdgcn_sched_barrier(0);
    });
    // wavefronts with fewer live fragments have fewer MFMAs to hide requests behind
    static_for<(NM + 1) / 2, 8>([&](auto rt) { read_y(rt); });
    static_for<((NM > 0 ? NM : 1) * ND) / 16, ND>([&](auto jt) { dma(jt); });
    __builtin_amdgcn_sched_barrier(0);
  };

  // ring state, in bytes from the start of the ring: units of the tile being multiplied
  // (sa, sw) and the two units the tile before it left free (fa, fw): W(kt+1) goes to fa,
  // A(kt+2) to fw
  auto next_slot = [](int s) { return s + 2 * kBigUnitBytes >= kBigUnits * kBigUnitBytes ? s + (2 - kBigUnits) * kBigUnitBytes : s + 2 * kBigUnitBytes; };
  int sa = 0, sw = kBigUnitBytes, fa = 3 * kBigUnitBytes, fw = 4 * kBigUnitBytes;
  const char* a2 = c.a_base + 2 * c.a_step;  // rows of A(kt+2)
  const char* w1 = c.w_base + c.w_step;      // rows of W(kt+1)

  // One K tile.  DO_W: W(kt+1)[4..7] is still to be requested; DO_A: A(kt+2) exists; NEXT:
  // a tile follows; NEXT_W: W(kt+2) exists.
  auto ktile = [&](auto do_w_tag, auto do_a_tag, auto next_tag, auto next_w_tag) {
    constexpr bool DO_W = decltype(do_w_tag)::value != 0, DO_A = decltype(do_a_tag)::value != 0;
    constexpr bool NEXT = decltype(next_tag)::value != 0, NEXT_W = decltype(next_w_tag)::value != 0;
    const uint32_t lds_fa = c.dma_lds + fa, lds_fw = c.dma_lds + fw;
    const char* const w2 = w1 + c.w_step;
    // request q of the tile's first STEPS-1 steps: W(kt+1)[4..7], then A(kt+2)[0..7]
    auto req = [&](auto qt) {
      constexpr int q = decltype(qt)::value;
      if constexpr (q < 4) { if constexpr (DO_W) lds_dma16_win<4 + q, q == 0>(w1, c.w_off[4 + q], lds_fa); }
      else { if constexpr (DO_A) lds_dma16_win<q - 4, q == 4>(a2, c.a_off[q - 4], lds_fw); }
    };
    using One = IntTag<1>;
    if constexpr (STEPS == 4) {
      step(IntTag<PER>{}, One{}, IntTag<1>{}, wfP, xfP, wfQ, xfQ, sa, sw, [&](auto jt) { req(jt); });
      step(IntTag<PER>{}, One{}, IntTag<2>{}, wfQ, xfQ, wfP, xfP, sa, sw, [&](auto jt) { req(IntTag<PER + decltype(jt)::value>{}); });
      step(IntTag<PER>{}, One{}, IntTag<3>{}, wfP, xfP, wfQ, xfQ, sa, sw, [&](auto jt) { req(IntTag<2 * PER + decltype(jt)::value>{}); });
    } else {
      step(IntTag<PER>{}, One{}, IntTag<1>{}, wfP, xfP, wfQ, xfQ, sa, sw, [&](auto jt) { req(jt); });
    }
    if constexpr (NEXT) {
      // tile kt+1 must have landed (only A(kt+2), the youngest request, may still be
      // outstanding) and nobody reads the slots of tile kt any more (its last fragment
      // reads have returned: lgkmcnt(0))
      if constexpr (DO_A) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      bare_barrier();
      fa = sa;
      fw = sw;
      sa = next_slot(sa);
      sw = next_slot(sw);
    }
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t lds_w2 = c.dma_lds + fa;  // W(kt+2) takes the token unit of the tile just finished
    step(IntTag<4>{}, IntTag<NEXT ? 1 : 0>{}, IntTag<0>{}, wfQ, xfQ, wfP, xfP, sa, sw, [&](auto it) {
      constexpr int i = decltype(it)::value;
      if constexpr (NEXT_W) lds_dma16_win<i, i == 0>(w2, c.w_off[i], lds_w2);
    });
    a2 += c.a_step;
    w1 += c.w_step;
  };

  // fill the ring: W(0) and half of W(1) were requested by the caller as soon as it knew
  // the expert; A(0) and A(1) follow here.  Then wait for tile 0 only.
  static_for<0, 8>([&](auto it) {
    constexpr int i = decltype(it)::value;
    lds_dma16_win<i, i == 0>(c.a_base, c.a_off[i], c.dma_lds);
  });
  if (1 < nk) {
    static_for<0, 8>([&](auto it) {
      constexpr int i = decltype(it)::value;
      lds_dma16_win<i, i == 0>(c.a_base + c.a_step, c.a_off[i], c.dma_lds + 2 * kBigUnitBytes);
    });
    wait_vmcnt<kBigDmaPerUnit>();
  } else {
    wait_vmcnt<0>();
  }
  bare_barrier();
  if constexpr (FMC > 0) {
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      const char* sta = smem + (sa + xl[ch]);
      const char* stw = smem + (sw + wl[ch]);
#pragma unroll
      for (int fn = 0; fn < 4; ++fn) wfP[fn][ch] = *reinterpret_cast<const uint4*>(stw + woff(fn));
#pragma unroll
      for (int fm = 0; fm < FMC; ++fm) xfP[fm][ch] = *reinterpret_cast<const uint4*>(sta + fm * 4096);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  using Yes = IntTag<1>;
  using No = IntTag<0>;
  for (int kt = 0; kt + 2 < nk; ++kt) ktile(Yes{}, Yes{}, Yes{}, Yes{});
  if (nk >= 2) ktile(Yes{}, No{}, Yes{}, No{});  // tile nk - 2: only the second half of W(nk-1) is still to come
  ktile(No{}, No{}, No{}, No{});                  // tile nk - 1
  wait_vmcnt<0>();
}

// Main loop for tiles with at most 64 real slots (an expert that received only a
// few rows): nothing but weight streaming, so the ring is laid out for that.
// Four 32 KB weight units (ring slots 1, 3, 0, 2 in that order, so that W(0) and
// W(1), requested by the caller before it knew the count, are where they
// belong) and four 8 KB token units of 64 rows inside slot 4.  Three K tiles are
// in flight while one is multiplied, twice what the general loop keeps in flight
// for weights, and a token unit costs two requests per wavefront instead of eight.
template <typename Mma, int FMC>
__device__ __forceinline__ void big_light_mainloop(const BigCtx& c, const char* smem, int nk,
                                                   f32x16 (&acc)[4][4]) {
  static_assert(FMC <= 2, "at most 64 token rows");
  constexpr int CH = Mma::kBigChunks, STEPS = 4 / CH;
  constexpr int kTokUnit = 2 * 4096;  // 64 rows
  auto w_slot = [](int k) {
    const int q = k & 3;
    return (q == 0 ? 1 : q == 1 ? 3 : q == 2 ? 0 : 2) * kBigUnitBytes;
  };
  auto a_slot = [](int k) { return 4 * kBigUnitBytes + (k & 3) * kTokUnit; };
  auto issue_w = [&](int k) {
    const char* const src = c.w_base + k * c.w_step;
    const uint32_t mid = c.dma_lds + w_slot(k);
    static_for<0, 8>([&](auto it) {
      constexpr int i = decltype(it)::value;
      lds_dma16_win<i, i == 0>(src, c.w_off[i], mid);
    });
  };
  // a token unit is 64 rows: the wavefront's window is 2 KB, two requests around its middle
  auto issue_a = [&](int k) {
    const char* const src = c.a_base + k * c.a_step;
    const uint32_t mid = c.dma_lds_light_a + (k & 3) * kTokUnit;
    lds_dma16_rel<-1024, true>(src, c.a_off[0], mid);
    lds_dma16_rel<0, false>(src, c.a_off[1], mid);
  };
  // request order: W(0) W(1) (first half by the caller) A(0) A(1) W(2) A(2), then W(k) A(k) per K tile
  if (1 < nk) {
    static_for<4, 8>([&](auto it) {
      constexpr int i = decltype(it)::value;
      lds_dma16_win<i, i == 4>(c.w_base + c.w_step, c.w_off[i], c.dma_lds + w_slot(1));
    });
  }
  issue_a(0);
  if (1 < nk) issue_a(1);
  if (2 < nk) { issue_w(2); issue_a(2); }
  for (int kt = 0; kt < nk; ++kt) {
    // unit kt has landed: only the (up to two) younger units may be outstanding; and
    // this wavefront is done reading unit kt-1, whose slots the next requests reuse
    const int left = nk - 1 - kt;
    if (kt == 0) {
      if (left >= 2) asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)" ::: "memory");
      else if (left == 1) asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    } else {
      if (left >= 2) asm volatile("s_waitcnt vmcnt(20) lgkmcnt(0)" ::: "memory");
      else if (left == 1) asm volatile("s_waitcnt vmcnt(10) lgkmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    }
    bare_barrier();
    if (kt + 3 < nk) { issue_w(kt + 3); issue_a(kt + 3); }
    if constexpr (FMC > 0) {
      const char* sw = smem + w_slot(kt);
      const char* sa = smem + a_slot(kt);
#pragma unroll
      for (int kk = 0; kk < STEPS; ++kk) {
        uint4 wf[4][CH], xf[FMC][CH];
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
#pragma unroll
          for (int fm = 0; fm < FMC; ++fm)
            xf[fm][ch] = *reinterpret_cast<const uint4*>(sa + fm * 32 * kBigRowBytes + c.rd_k[kk * CH + ch]);
#pragma unroll
          for (int fn = 0; fn < 4; ++fn)
            wf[fn][ch] = *reinterpret_cast<const uint4*>(sw + c.w_row[fn] + c.rd_k[kk * CH + ch]);
        }
#pragma unroll
        for (int fm = 0; fm < FMC; ++fm)
#pragma unroll
          for (int fn = 0; fn < 4; ++fn) acc[fn][fm] = Mma::mma_big(wf[fn], xf[fm], acc[fn][fm]);
      }
    }
  }
  wait_vmcnt<0>();
}

template <typename El>
__device__ __forceinline__ float unpack_lo(uint32_t w);
template <typename El>
__device__ __forceinline__ float unpack_hi(uint32_t w);
template <>
__device__ __forceinline__ float unpack_lo<ElemBF16>(uint32_t w) { return __uint_as_float(w << 16); }
template <>
__device__ __forceinline__ float unpack_hi<ElemBF16>(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
template <>
__device__ __forceinline__ float unpack_lo<ElemF16>(uint32_t w) { return f16_bits_to_f32(static_cast<uint16_t>(w)); }
template <>
__device__ __forceinline__ float unpack_hi<ElemF16>(uint32_t w) { return f16_bits_to_f32(static_cast<uint16_t>(w >> 16)); }

template <typename El, int ACT>
__device__ __forceinline__ uint32_t gated_pair(const GemmParams& p, uint32_t gw, uint32_t uw) {
  const float g0 = unpack_lo<El>(gw), g1 = unpack_hi<El>(gw);
  const float u0 = unpack_lo<El>(uw), u1 = unpack_hi<El>(uw);
  if constexpr (ACT == MOE_ACT_SWIGLUOAI) {
    return pack2<El>(moe_swigluoai(g0, u0, p.alpha, p.limit), moe_swigluoai(g1, u1, p.alpha, p.limit));
  } else {
    float a0, a1;
    if constexpr (ACT == MOE_ACT_SILU) {
      a0 = silu_fast(g0);
      a1 = silu_fast(g1);
    } else {
      a0 = 0.5f * g0 * (1.f + erff(g0 * 0.70710678118654752f));
      a1 = 0.5f * g1 * (1.f + erff(g1 * 0.70710678118654752f));
    }
    const uint32_t aw = pack2<El>(a0, a1);  // the activation is stored in T before the product
    return pack2<El>(unpack_lo<El>(aw) * u0, unpack_hi<El>(aw) * u1);
  }
}

// Epilogue phase 1: park this wavefront's results in its LDS window as
// [token row][weight row], rounded to the activation dtype after the optional
// scales, bias and routed weight.  FAST_SILU (gated pass with SiLU): gate row n
// and up row n of the weight unit are the same accumulator element of fragments
// fn and fn + 2, so silu(gate) * up is formed here on the fp32 values (hardware
// exp2/rcp, one rounding at the end) and only the 64 output columns are parked.
// The other activations park gate and up rounded, as the stand-alone activation
// kernels see them, and the flush combines them.
template <typename El, int FMC, bool GATED, bool SCALED, bool BIAS, bool FAST_SILU>
__device__ __forceinline__ void big_park(const GemmParams& p, int e, int n0, int wn, int lhi, int l32,
                                         const float* s_rw, const float* s_as, const float* s_ws,
                                         const float* s_bias, char* epi, const f32x16 (&acc)[4][4]) {
  // e4m3: the accumulator is in units of (row scale of the A operand) x (weight row scale).
  // Scales and biases of the weight rows were put into LDS in the order of the weight unit's rows.
  [[maybe_unused]] int ws_row[4];
#pragma unroll
  for (int fn = 0; fn < 4; ++fn) {
    if constexpr (GATED) ws_row[fn] = (fn < 2) ? wn * 64 + fn * 32 : 128 + wn * 64 + (fn - 2) * 32;
    else ws_row[fn] = wn * 128 + fn * 32;
  }
  // four consecutive accumulator elements of fragment fn, scaled, biased, weighted
  auto load4 = [&](int fn, int fm, int g, float as, float rw, float (&v)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = acc[fn][fm][4 * g + i];
    if constexpr (SCALED) {
      const float4 w4 = *reinterpret_cast<const float4*>(s_ws + ws_row[fn] + 8 * g + 4 * lhi);
      v[0] *= as * w4.x; v[1] *= as * w4.y; v[2] *= as * w4.z; v[3] *= as * w4.w;
    }
    if constexpr (BIAS) {
      const float4 b4 = *reinterpret_cast<const float4*>(s_bias + ws_row[fn] + 8 * g + 4 * lhi);
      v[0] += b4.x; v[1] += b4.y; v[2] += b4.z; v[3] += b4.w;
    }
    // rw is exactly 1 when the routed weight is not applied in this pass
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] *= rw;
  };
#pragma unroll
  for (int fm = 0; fm < FMC; ++fm) {
    const float rw = s_rw[fm * 32 + l32];
    [[maybe_unused]] const float as = SCALED ? s_as[fm * 32 + l32] : 1.f;
    char* row = epi + (fm * 32 + l32) * kEpiRowBytes;
#pragma unroll
    for (int fn = 0; fn < (FAST_SILU ? 2 : 4); ++fn) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float v[4];
        load4(fn, fm, g, as, rw, v);
        if constexpr (FAST_SILU) {
          float u[4];
          load4(fn + 2, fm, g, as, rw, u);
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = silu_fast(v[i]) * u[i];
        }
        *reinterpret_cast<uint2*>(row + (fn * 32 + 8 * g + 4 * lhi) * 2) =
            uint2{pack2<El>(v[0], v[1]), pack2<El>(v[2], v[3])};
      }
    }
  }
}

// Epilogue phase 2: write the parked tile to global memory, 8 columns (16 bytes)
// per lane and step.  After a gated pass with SiLU the 64 output columns of a
// row are parked ready; with the other activations columns [0,64) of a row are
// gate values and [64,128) the matching up values, combined here.
template <typename El, bool GATED, int ACT>
__device__ __forceinline__ void big_flush(const GemmParams& p, int n0, int wn, int lane, int slot0,
                                          int rows, const int* s_tok, const char* epi) {
  using S = typename El::S;
  constexpr int COLS = GATED ? 64 : 128;      // output columns of the wavefront tile
  constexpr int LPR = COLS / 8;               // lanes per row
  constexpr int RPS = kWave / LPR;            // rows per step
  constexpr bool PAIRS = GATED && ACT != MOE_ACT_SILU;  // gate and up parked side by side, activation applied here
  constexpr int UNR = PAIRS ? 4 : 8;          // steps in flight: LDS reads, math and stores overlap
  const int c8 = (lane % LPR) * 8;
  const int ncol = n0 + wn * COLS + c8;
  const bool vec_ok = ncol + 7 < p.N && (p.ldc & 7) == 0;
  // The gate-up result as 32 KB units of the down pass's A operand: this wavefront's 64 columns
  // are K tile 2 * (n-tile) + wn of the block, its rows 128 bytes each, chunks in LDS order.
  // N is a multiple of 64 then, so a wavefront is inside the matrix or has nothing to write.
  bool tiled = false;
  if constexpr (GATED) tiled = p.c_tiled != 0;
  if (tiled && n0 + wn * COLS >= p.N) return;
  // Whole wavefront inside the matrix: no per-lane edge handling.  Real slots come
  // first in a block, so row r is live exactly when r < rows.
  if (tiled || (n0 + wn * COLS + COLS <= p.N && (p.ldc & 7) == 0)) {
    const int lrow = lane / LPR;
    char* cbase = static_cast<char*>(p.c) + static_cast<int64_t>(ncol) * 2;
    int64_t ldc_bytes = static_cast<int64_t>(p.ldc) * 2;
    if (tiled) {
      const int64_t unit = static_cast<int64_t>(slot0 >> 8) * (p.N >> 6) + (n0 >> 6) + wn;
      cbase = static_cast<char*>(p.c) + unit * kBigUnitBytes;
      ldc_bytes = kBigRowBytes;
    }
    const char* src = epi + lrow * kEpiRowBytes + c8 * 2;
    for (int r0 = 0; r0 < rows; r0 += RPS * UNR) {
      int crow[UNR];
      uint4 gq[UNR], uq[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int r = r0 + u * RPS + lrow;  // < 128: rows <= 128 and 128 is a multiple of RPS * UNR
        crow[u] = p.a_by_slot ? s_tok[r] : slot0 + r;
        if (tiled) {
          const int rb = (slot0 & 255) + r;  // row inside the block; the row's byte offset carries the chunk
          crow[u] = rb;
        }
        gq[u] = *reinterpret_cast<const uint4*>(src + (r0 + u * RPS) * kEpiRowBytes);
        if constexpr (PAIRS) uq[u] = *reinterpret_cast<const uint4*>(src + (r0 + u * RPS) * kEpiRowBytes + 128);
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        uint4 out = gq[u];
        if constexpr (PAIRS)
          out = uint4{gated_pair<El, ACT>(p, gq[u].x, uq[u].x), gated_pair<El, ACT>(p, gq[u].y, uq[u].y),
                      gated_pair<El, ACT>(p, gq[u].z, uq[u].z), gated_pair<El, ACT>(p, gq[u].w, uq[u].w)};
        if (r0 + u * RPS + lrow < rows) {
          char* dst = cbase + crow[u] * ldc_bytes;
          if (tiled) dst += ((lane & 7) ^ ((crow[u] >> 1) & 7)) << 4;
          if (p.wt_stores) store16_device_scope(dst, out);
          else *reinterpret_cast<uint4*>(dst) = out;
        }
      }
    }
    return;
  }
  for (int r0 = 0; r0 < rows; r0 += RPS * UNR) {
    int tok[UNR];
    uint4 gq[UNR], uq[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int r = r0 + u * RPS + lane / LPR;
      tok[u] = r < rows ? s_tok[r] : p.numel;
      const char* row = epi + (r < 128 ? r : 127) * kEpiRowBytes;
      gq[u] = *reinterpret_cast<const uint4*>(row + c8 * 2);
      if constexpr (PAIRS) uq[u] = *reinterpret_cast<const uint4*>(row + (64 + c8) * 2);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      if (tok[u] >= p.numel) continue;
      uint4 out = gq[u];
      if constexpr (PAIRS)
        out = uint4{gated_pair<El, ACT>(p, gq[u].x, uq[u].x), gated_pair<El, ACT>(p, gq[u].y, uq[u].y),
                    gated_pair<El, ACT>(p, gq[u].z, uq[u].z), gated_pair<El, ACT>(p, gq[u].w, uq[u].w)};
      const int slot = slot0 + r0 + u * RPS + lane / LPR;
      const int64_t crow = p.a_by_slot ? tok[u] : slot;
      S* dst = static_cast<S*>(p.c) + crow * p.ldc + ncol;
      if (vec_ok) {
        *reinterpret_cast<uint4*>(dst) = out;
      } else {
        const uint32_t w4[4] = {out.x, out.y, out.z, out.w};
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (ncol + i < p.N) dst[i] = static_cast<S>(w4[i >> 1] >> (16 * (i & 1)));
      }
    }
  }
}

template <typename Mma, int FMC, bool GATED, bool LIGHT = false>
__device__ __forceinline__ void big_wave(const GemmParams& p, const BigCtx& c, char* smem, int nk,
                                         int e, int n0, int wn, int wm, int lane, int my_tok, float my_rw,
                                         float my_as, float my_ws, float my_bias, int* s_tok_all, float* s_rw_all, char* epi) {
  using El = typename Mma::El;
  f32x16 acc[4][4];
#pragma unroll
  for (int fn = 0; fn < 4; ++fn)
#pragma unroll
    for (int fm = 0; fm < 4; ++fm)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[fn][fm][r] = 0.f;
  if constexpr (LIGHT) {
    big_light_mainloop<Mma, FMC>(c, smem, nk, acc);
  } else {
    big_mainloop<Mma, FMC, GATED>(c, smem, nk, acc);
  }
  bare_barrier();  // every wavefront is done reading the ring before it is reused
  s_tok_all[threadIdx.x] = my_tok;
  s_rw_all[threadIdx.x] = my_rw;  // requested before the main loop, needed only now
  s_rw_all[kBigBM + threadIdx.x] = my_as;
  s_rw_all[2 * kBigBM + threadIdx.x] = my_ws;
  s_rw_all[3 * kBigBM + threadIdx.x] = my_bias;
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  bare_barrier();
  if constexpr (FMC > 0) {
    // one straight-line body per case: a test per element costs more than the element
    auto park = [&](auto bias_tag, auto silu_tag) {
      big_park<El, FMC, GATED, Mma::kEs == 1, decltype(bias_tag)::value != 0, decltype(silu_tag)::value != 0>(
          p, e, n0, wn, lane >> 5, lane & 31, s_rw_all + wm * 128, s_rw_all + kBigBM + wm * 128,
          s_rw_all + 2 * kBigBM, s_rw_all + 3 * kBigBM, epi, acc);
    };
    bool fast_silu = false;
    if constexpr (GATED) fast_silu = p.activation == MOE_ACT_SILU;
    if constexpr (GATED) {
      if (fast_silu) {
        if (p.bias) park(IntTag<1>{}, IntTag<1>{});
        else park(IntTag<0>{}, IntTag<1>{});
      }
    }
    if (!fast_silu) {
      if (p.bias) park(IntTag<1>{}, IntTag<0>{});
      else park(IntTag<0>{}, IntTag<0>{});
    }
  }
}

// One output tile of the large-tile kernel: m-block mb, n-tile nt.
template <typename Mma, bool GATED>
__device__ __forceinline__ void big_tile(const GemmParams& p, int mb, int nt, char* smem) {
  using El = typename Mma::El;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lhi = lane >> 5;
  const int wm = wave & 1, wn = wave >> 1;
  // the two loads below do not depend on each other: one memory latency, not two
  const int e = __builtin_amdgcn_readfirstlane(p.expert_ids[(mb * kBigBM) / p.align_bs]);
  const int64_t my_slot = static_cast<int64_t>(mb) * kBigBM + tid;
  const int my_tok = p.sorted_ids[my_slot < p.sorted_cap ? my_slot : p.sorted_cap - 1];
  const int n0 = nt * (GATED ? kBigBNW / 2 : kBigBNW);
  int* s_tok = reinterpret_cast<int*>(smem + kBigLdsBytes);
  float* s_rw_all = reinterpret_cast<float*>(smem + kBigLdsBytes + kBigBM * 4);
  s_tok[tid] = my_tok;
  // real slots come first in a block: count them (dynamic LDS only, the ring needs all 160 KB)
  int* s_cnt = reinterpret_cast<int*>(smem + kBigLdsBytes + kBigSideBytes);
  const int wave_cnt = __popcll(__ballot(my_tok < p.numel));
  if (lane == 0) s_cnt[wave] = wave_cnt;
  constexpr int ES = Mma::kEs, CH = Mma::kBigChunks;
  const int nk = p.Kd / (kBigRowBytes / ES);
  BigCtx c;
  // DMA geometry: wavefront w fills bytes [8192 w, 8192 w + 8192) of every unit with eight requests
  // of 1 KB; request j of lane l is unit row 64 w + 8 j + l / 8, position l % 8 of that row, which
  // holds the row's 16-byte chunk (l % 8) ^ ((row >> 1) & 7).  The base pointers are 4096 short of
  // the operands (dma_win_bias).
  const int dma_row0 = 64 * wave + (lane >> 3);
  auto dma_chunk = [&](int row) { return (lane & 7) ^ ((row >> 1) & 7); };
  c.a_base = static_cast<const char*>(p.a) - 4096;
  c.w_base = static_cast<const char*>(p.w) + static_cast<int64_t>(e) * p.w_stride_e * ES - 4096;
  c.dma_lds = __builtin_amdgcn_readfirstlane(lds_offset_of(smem) + wave * 8192 + 4096);
  c.dma_lds_light_a = __builtin_amdgcn_readfirstlane(lds_offset_of(smem) + 4 * kBigUnitBytes + wave * 2048 + 1024);
  c.a_step = c.w_step = kBigRowBytes;
  if (p.w_tiled) {
    // unit (n-tile, K tile) of this expert is one 32 KB piece in LDS order: every request reads
    // the bytes it writes
    c.w_base += static_cast<int64_t>(nt) * nk * kBigUnitBytes;
    c.w_step = kBigUnitBytes;
#pragma unroll
    for (int i = 0; i < 8; ++i) c.w_off[i] = static_cast<uint32_t>(wave * 8192 + i * 1024 + lane * 16) + dma_win_bias(i);
  } else {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int rr = dma_row0 + 8 * i;
    int64_t wrow;
    if constexpr (GATED) {
      const int half = rr >> 7;
      int n = n0 + (rr & 127);
      n = n < p.N ? n : p.N - 1;
      wrow = p.interleaved ? (2 * n + half) : (half * p.N + n);
    } else {
      const int n = n0 + rr;
      wrow = n < p.N ? n : p.N - 1;
    }
    c.w_off[i] = static_cast<uint32_t>(wrow * p.w_stride_n * ES + dma_chunk(rr) * 16) + dma_win_bias(i);
  }
  }
  // The weights of the first K tile and a half are on their way (ring slots 1 and 3) while
  // the slot ids are still being looked at: they are the cold half of the fill.
  // Neither slot overlaps the side arrays above.
  static_for<0, 8>([&](auto it) {
    constexpr int i = decltype(it)::value;
    lds_dma16_win<i, i == 0>(c.w_base, c.w_off[i], c.dma_lds + kBigUnitBytes);
  });
  if (1 < nk) {  // the first half of W(1); the main loops request the second
    static_for<0, 4>([&](auto it) {
      constexpr int i = decltype(it)::value;
      lds_dma16_win<i, i == 0>(c.w_base + c.w_step, c.w_off[i], c.dma_lds + 3 * kBigUnitBytes);
    });
  }
  __syncthreads();
  const int nvalid = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
  if (nvalid == 0) {
    wait_vmcnt<0>();  // nothing may still be landing in LDS when the workgroup ends
    return;
  }
  float my_rw = 1.f, my_as = 1.f, my_ws = 1.f;
  if (p.mul_weight) my_rw = my_tok < p.numel ? p.topk_w[my_tok] : 0.f;
  if (p.a_scale && my_tok < p.numel) my_as = p.a_scale[p.a_by_slot ? my_slot : my_tok / p.top_k];
  float my_bias = 0.f;
  if (p.w_scale || p.bias) {
    // scale and bias of the weight row that sits at row `tid` of a weight unit
    int64_t wr;
    if constexpr (GATED) {
      int n = n0 + (tid & 127);
      n = n < p.N ? n : p.N - 1;
      wr = p.interleaved ? (2 * n + (tid >> 7)) : ((tid >> 7) * p.N + n);
    } else {
      wr = n0 + tid < p.N ? n0 + tid : p.N - 1;
    }
    if (p.w_scale) my_ws = p.w_scale[e * p.w_scale_stride_e + wr];
    if (p.bias) my_bias = El::ld(static_cast<const typename El::S*>(p.bias)[e * p.bias_stride_e + wr]);
  }
  if (p.a_tiled) {
    // the block's rows of K tile kt are unit (mb, kt), written in LDS order by the gate-up pass
    c.a_base += static_cast<int64_t>(mb) * nk * kBigUnitBytes;
    c.a_step = kBigUnitBytes;
  }
  // A weight-streaming tile (at most 64 real slots) loads token units of 64 rows: there the
  // wavefront's window is 2 KB, rows 16 w + 8 j + l / 8, two requests with the offsets -1024 and 0.
  const bool light_a = nvalid <= 64;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int row = light_a ? 16 * wave + 8 * (i & 1) + (lane >> 3) : dma_row0 + 8 * i;
    const uint32_t bias = light_a ? static_cast<uint32_t>(4096 - ((i & 1) - 1) * 1024) : dma_win_bias(i);
    // a request whose eight rows are all padding asks for rows 0..7 again (an L1 hit), so that
    // every token unit is the same number of loads and the vmcnt bookkeeping stays fixed
    const bool dead = (row & ~7) >= nvalid;
    const int pos_row = row;   // the row whose place in LDS the data takes (it decides the chunk order)
    if (dead) row = lane >> 3;
    if (p.a_tiled) {
      // (a dead request reads the bytes of live rows 0..7 into its own place: never looked at)
      c.a_off[i] = static_cast<uint32_t>(row * kBigRowBytes + (lane & 7) * 16) + bias;
      continue;
    }
    int64_t src = static_cast<int64_t>(mb) * kBigBM + row;
    if (!p.a_by_slot) {
      const int tok = s_tok[row];
      src = tok < p.numel ? tok / p.top_k : 0;
    }
    c.a_off[i] = static_cast<uint32_t>(src * p.lda * ES + dma_chunk(pos_row) * 16) + bias;
  }
  // chunk ch of MFMA step kk: lane half lhi owns the K elements of chunks CH * (2 kk + lhi) .. + CH - 1
#pragma unroll
  for (int q = 0; q < 4; ++q)
    c.rd_k[q] = l32 * kBigRowBytes + (((CH * (2 * (q / CH) + lhi) + q % CH) ^ ((l32 >> 1) & 7)) << 4);
  c.x_row = wm * 128 * kBigRowBytes;
#pragma unroll
  for (int fn = 0; fn < 4; ++fn) {
    int r;
    if constexpr (GATED)
      r = (fn < 2) ? wn * 64 + fn * 32 : 128 + wn * 64 + (fn - 2) * 32;
    else
      r = wn * 128 + fn * 32;
    c.w_row[fn] = r * kBigRowBytes;
  }
  const int slot0 = mb * kBigBM + wm * 128;
  char* epi = smem + wave * kEpiWaveBytes;
  const int rows = min(128, max(0, nvalid - wm * 128));  // real slots of this wavefront
  __syncthreads();  // s_tok sits inside the ring: everyone has read it before any DMA may land there
  if (nvalid <= 64) {
    // a workgroup-wide choice: every wavefront runs the streaming-shaped loop
    switch ((rows + 31) >> 5) {
      case 0: big_wave<Mma, 0, GATED, true>(p, c, smem, nk, e, n0, wn, wm, lane, my_tok, my_rw, my_as, my_ws, my_bias, s_tok, s_rw_all, epi); break;
      case 1: big_wave<Mma, 1, GATED, true>(p, c, smem, nk, e, n0, wn, wm, lane, my_tok, my_rw, my_as, my_ws, my_bias, s_tok, s_rw_all, epi); break;
      default: big_wave<Mma, 2, GATED, true>(p, c, smem, nk, e, n0, wn, wm, lane, my_tok, my_rw, my_as, my_ws, my_bias, s_tok, s_rw_all, epi); break;
    }
  } else
  switch ((rows + 31) >> 5) {
    case 0: big_wave<Mma, 0, GATED>(p, c, smem, nk, e, n0, wn, wm, lane, my_tok, my_rw, my_as, my_ws, my_bias, s_tok, s_rw_all, epi); break;
    case 1: big_wave<Mma, 1, GATED>(p, c, smem, nk, e, n0, wn, wm, lane, my_tok, my_rw, my_as, my_ws, my_bias, s_tok, s_rw_all, epi); break;
    case 2: big_wave<Mma, 2, GATED>(p, c, smem, nk, e, n0, wn, wm, lane, my_tok, my_rw, my_as, my_ws, my_bias, s_tok, s_rw_all, epi); break;
    case 3: big_wave<Mma, 3, GATED>(p, c, smem, nk, e, n0, wn, wm, lane, my_tok, my_rw, my_as, my_ws, my_bias, s_tok, s_rw_all, epi); break;
    default: big_wave<Mma, 4, GATED>(p, c, smem, nk, e, n0, wn, wm, lane, my_tok, my_rw, my_as, my_ws, my_bias, s_tok, s_rw_all, epi); break;
  }
  if constexpr (GATED) {
    if (p.activation == MOE_ACT_SILU)
      big_flush<El, true, MOE_ACT_SILU>(p, n0, wn, lane, slot0, rows, s_tok + wm * 128, epi);
    else if (p.activation == MOE_ACT_SWIGLUOAI)
      big_flush<El, true, MOE_ACT_SWIGLUOAI>(p, n0, wn, lane, slot0, rows, s_tok + wm * 128, epi);
    else
      big_flush<El, true, MOE_ACT_GELU>(p, n0, wn, lane, slot0, rows, s_tok + wm * 128, epi);
  } else {
    big_flush<El, false, MOE_ACT_SILU>(p, n0, wn, lane, slot0, rows, s_tok + wm * 128, epi);
  }
}

template <typename Mma, bool GATED>
__global__ __launch_bounds__(kThreads, 1) void big_gemm_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // only the m-blocks below the padded total are live: cut the per-XCD ranges from
  // those, so that no XCD is left holding the grid's empty tail
  const int xslot = blockIdx.x / kXcds;
  int nt, mb;
  if (p.xcd_bounds) {
    // ranges of equal estimated work (big_plan_kernel), m-block major inside a range
    const int lo = p.xcd_bounds[blockIdx.x % kXcds], hi = p.xcd_bounds[blockIdx.x % kXcds + 1];
    mb = lo + xslot / p.num_n_tiles;
    nt = xslot % p.num_n_tiles;
    // the second test keeps a plan that was never written from sending a tile out of range
    if (mb >= hi || lo < 0 || mb >= p.num_m_blocks) return;
  } else {
  const int npp = *p.num_post_pad;
  const int live_mb = (npp + kBigBM - 1) / kBigBM;
  const int live = live_mb * p.num_n_tiles;
  const int per_xcd = (live + kXcds - 1) / kXcds;
  const int logical = (blockIdx.x % kXcds) * per_xcd + xslot;
  if (xslot >= per_xcd || logical >= live) return;
  if (p.m_major) {
    mb = logical / p.num_n_tiles;
    nt = logical - mb * p.num_n_tiles;
  } else {
    nt = logical / live_mb;
    mb = logical - nt * live_mb;
  }
  }
  big_tile<Mma, GATED>(p, mb, nt, smem);
}

// Both passes in one launch, for the 16-bit dtypes.  Workgroup ids go to the XCDs
// round robin and an XCD starts its workgroups in id order: each XCD first gets
// the gate-up tiles of its m-block range, then the down tiles of the same range,
// so its CUs move on to down tiles while the last gate-up tiles are still running
// instead of idling through the tail of one launch and the ramp of the next.
// done[mb] counts the finished gate-up tiles of m-block mb (zeroed by the plan
// step); a down tile starts once all of them are in, which at its place in the
// order is normally long the case.  The hand-off holds at device scope: the
// gate-up workgroup's results leave as write-through stores (sc1) and are
// complete before its count goes up, and the down tile's loads come after an
// acquire fence behind the full count, so the result does not depend on which
// XCD either side ran on.
// The wait is bounded (spin_limit polls of about a microsecond) so that the grid
// drains whatever happens.  A down tile whose wait expires does not multiply a
// partly written intermediate: it fills its output rows with NaN, which the top-k
// combine carries into `out`, and adds one to the status word that
// moe_fused_experts_status reads back.
template <typename El>
__device__ __forceinline__ void big_poison_tile(const GemmParams& p, int mb, int nt) {
  using S = typename El::S;
  const int64_t slot = static_cast<int64_t>(mb) * kBigBM + threadIdx.x;
  if (slot >= p.sorted_cap) return;
  const int tok = p.sorted_ids[slot];
  if (tok >= p.numel) return;
  const S nan = sizeof(S) == 2 ? El::st(__builtin_nanf("")) : S{};
  S* row = static_cast<S*>(p.c) + static_cast<int64_t>(tok) * p.ldc;
  const int n0 = nt * kBigBNW;
  for (int n = n0; n < n0 + kBigBNW && n < p.N; ++n) row[n] = nan;
}

template <typename Mma>
__global__ __launch_bounds__(kThreads, 1) void big_fused_kernel(const GemmParams p1, const GemmParams p2,
                                                                int32_t* __restrict__ done, int cap_mb,
                                                                int spin_limit, int32_t* __restrict__ status,
                                                                int down_xcd_shift) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int xslot = blockIdx.x / kXcds;
  const int n1 = cap_mb * p1.num_n_tiles;
  // down_xcd_shift != 0 (a test setting): the down tiles of XCD x take the m-block range of XCD
  // x + shift, so that every hand-off crosses from one XCD's L2 to another's.  Gate-up tiles never
  // wait and precede the down tiles in every XCD's list, so the grid still drains.
  const int x = (blockIdx.x % kXcds + (xslot < n1 ? 0 : down_xcd_shift)) % kXcds;
  const int lo = p1.xcd_bounds[x], hi = p1.xcd_bounds[x + 1];
  if (xslot < n1) {
    const int mb = lo + xslot / p1.num_n_tiles, nt = xslot % p1.num_n_tiles;
    if (mb >= hi || lo < 0 || mb >= p1.num_m_blocks) return;  // (an unwritten plan must not send a tile out of range)
    big_tile<Mma, true>(p1, mb, nt, smem);
    // Every store of this workgroup is complete before the barrier.  With write-through stores
    // (whole tiles inside the matrix) that means visible device-wide; otherwise the release
    // writes the L2 back first.  Measured at 8448 tokens, both passes: 766 us with no ordering
    // at all, 772 us this way, 826 us with the write-back on every tile.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      if (p1.wt_stores) __hip_atomic_fetch_add(done + mb, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else __hip_atomic_fetch_add(done + mb, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    }
  } else {
    const int j = xslot - n1;
    const int mb = lo + j / p2.num_n_tiles, nt = j % p2.num_n_tiles;
    if (mb >= hi || lo < 0 || mb >= p1.num_m_blocks) return;
    int* s_flag = reinterpret_cast<int*>(smem + kBigLdsBytes + kBigSideBytes + 16);
    if (threadIdx.x == 0) {
      int spins = 0;
      bool ready;
      while (!(ready = __hip_atomic_load(done + mb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= p1.num_n_tiles) &&
             spins++ < spin_limit)
        __builtin_amdgcn_s_sleep(32);
      *s_flag = ready ? 1 : 0;
    }
    __syncthreads();
    // Every wavefront orders its own loads of the block's rows behind the count it has just been told
    // of: the acquire fence drops the cached lines (and completes, vmcnt(0)) in the wavefront that
    // issues it, and a workgroup barrier alone does not extend that to the other three.
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (*s_flag == 0) {  // workgroup-uniform
      big_poison_tile<typename Mma::El>(p2, mb, nt);
      if (threadIdx.x == 0) __hip_atomic_fetch_add(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    // (the flag word lies behind the epilogue's staging area and side arrays, in the ring's last unit,
    // which big_tile writes only behind its own barriers)
    big_tile<Mma, false>(p2, mb, nt, smem);
  }
}


// Cuts the live m-blocks of a large-tile launch into one contiguous range per XCD
// with equal estimated work instead of equal counts.  A block of an expert that
// received at most 32 (64) rows is weight streaming only and costs about 0.60
// (0.75) of a full one, a partly filled one as much as a full one (its six gate-up
// and eight down tiles: 334 / 424 / 568 / 561 us of CU time at 8448 tokens); with
// equal counts the XCDs finished up to 25 % apart.
// Ranges stay contiguous so that the blocks of one expert keep sharing its
// weights through one L2.  No range is longer than cap_mb blocks (the grid has
// that many slots per XCD).  One workgroup; bounds[0..8] in m-blocks.
constexpr int kPlanThreads = 1024;
__global__ __launch_bounds__(kPlanThreads) void big_plan_kernel(const int32_t* __restrict__ sorted_ids,
                                                                const int32_t* __restrict__ num_post_pad,
                                                                int numel, int cap_mb, int32_t* __restrict__ bounds,
                                                                int32_t* __restrict__ done, int num_done) {
  __shared__ int s_wave[kPlanThreads / kWave + 1];
  // per-m-block counters of the one-launch form start at zero, and so does the count of expired waits
  for (int i = threadIdx.x; i < num_done; i += kPlanThreads) done[i] = 0;
  if (threadIdx.x == 0) bounds[kBigStatusWord] = 0;
  __shared__ int s_b[kXcds + 1];
  const int live_mb = (*num_post_pad + kBigBM - 1) / kBigBM;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  auto weight = [&](int mb) {
    if (mb >= live_mb) return 0;
    const int32_t* s = sorted_ids + static_cast<int64_t>(mb) * kBigBM;
    return s[32] >= numel ? 38 : (s[64] >= numel ? 48 : 64);
  };
  // inclusive scan of `v` over the workgroup, plus the workgroup total
  auto scan = [&](int v, int& total) {
    int inc = v;
#pragma unroll
    for (int d = 1; d < kWave; d *= 2) {
      const int o = __shfl_up(inc, d, kWave);
      if (lane >= d) inc += o;
    }
    __syncthreads();
    if (lane == kWave - 1) s_wave[wave] = inc;
    __syncthreads();
    if (threadIdx.x == 0) {
      int run = 0;
      for (int w = 0; w < kPlanThreads / kWave; ++w) { const int t = s_wave[w]; s_wave[w] = run; run += t; }
      s_wave[kPlanThreads / kWave] = run;
    }
    __syncthreads();
    total = s_wave[kPlanThreads / kWave];
    return inc + s_wave[wave];
  };
  int total = 0;
  for (int base = 0; base < live_mb; base += kPlanThreads) {
    int t;
    scan(weight(base + threadIdx.x), t);
    total += t;
  }
  if (threadIdx.x <= kXcds) s_b[threadIdx.x] = threadIdx.x == 0 ? 0 : live_mb;
  __syncthreads();
  int before = 0;
  for (int base = 0; base < live_mb; base += kPlanThreads) {
    const int mb = base + threadIdx.x;
    const int w = weight(mb);
    int t;
    const int inc = before + scan(w, t), exc = inc - w;
    if (w > 0) {
      // the block whose cost takes the running sum across x / 8 of the total is the last of XCD x - 1
#pragma unroll
      for (int x = 1; x < kXcds; ++x) {
        const int64_t target = (static_cast<int64_t>(total) * x + kXcds - 1) / kXcds;
        if (exc < target && inc >= target) s_b[x] = mb + 1;
      }
    }
    before += t;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    // a total of 0 (no live block) leaves every bound at live_mb = 0; otherwise bounds ascend
    for (int x = 1; x <= kXcds; ++x) s_b[x] = max(s_b[x], s_b[x - 1]);
    for (int x = 1; x <= kXcds; ++x) s_b[x] = min(s_b[x], s_b[x - 1] + cap_mb);
    s_b[kXcds] = live_mb;
    for (int x = kXcds - 1; x >= 1; --x) s_b[x] = max(s_b[x], s_b[x + 1] - cap_mb);
    for (int x = 0; x <= kXcds; ++x) bounds[x] = s_b[x];
  }
}

// Epilogue of the streaming kernel for full, aligned 16-bit tiles: same storage
// points as store_fragment, with the hardware conversions and the fast SiLU of
// the large-tile epilogue (one wavefront finishes the whole tile, so the
// instruction count is the epilogue's latency).
template <typename El, bool GATED, int ACT>
__device__ __forceinline__ void stream_store(const GemmParams& p, int e, const f32x16& ga, const f32x16& ua,
                                             int tok, int slot, int ncol0, float rw) {
  using S = typename El::S;
  const S* bias = static_cast<const S*>(p.bias);
  const int64_t crow = p.a_by_slot ? tok : slot;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int n = ncol0 + 8 * g;
    float gv[4], uv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      gv[i] = ga[4 * g + i];
      uv[i] = ua[4 * g + i];
      if (bias) {
        if constexpr (GATED) {
          gv[i] += El::ld(bias[e * p.bias_stride_e + (p.interleaved ? 2 * (n + i) : n + i)]);
          uv[i] += El::ld(bias[e * p.bias_stride_e + (p.interleaved ? 2 * (n + i) + 1 : p.N + n + i)]);
        } else {
          gv[i] += El::ld(bias[e * p.bias_stride_e + n + i]);
        }
      }
      gv[i] *= rw;
      uv[i] *= rw;
    }
    uint2 out;
    if constexpr (GATED) {
      out.x = gated_pair<El, ACT>(p, pack2<El>(gv[0], gv[1]), pack2<El>(uv[0], uv[1]));
      out.y = gated_pair<El, ACT>(p, pack2<El>(gv[2], gv[3]), pack2<El>(uv[2], uv[3]));
    } else {
      out.x = pack2<El>(gv[0], gv[1]);
      out.y = pack2<El>(gv[2], gv[3]);
    }
    *reinterpret_cast<uint2*>(static_cast<S*>(p.c) + crow * p.ldc + n) = out;
  }
}

// ---------------------------------------------------------------------------
// Streaming variant for bandwidth-bound calls (a few tokens per expert: decode).
// The time of such a call is the time to pull every active expert's weights
// out of HBM once, so the kernel is built around that stream: a workgroup owns
// 64 weight rows of one expert and one alignment block of 32 slots, and walks
// K in units of 64 elements.  A unit (64 weight rows and 32 token rows of
// 128 B: 8 KB + 4 KB) goes global->LDS by DMA into a ring of four units, three
// of them in flight while the fourth is multiplied; three workgroups fit a CU,
// which keeps about 100 KB per CU on its way from HBM and hides a workgroup's
// start-up and epilogue behind its neighbours' streams.  Small tiles (256 KB of
// weights in the gate-up pass) also keep the last wave of workgroups short.
// All four wavefronts issue DMA requests; the MFMA work of a 32-slot block is
// so small (8 MFMAs per unit) that wavefront 0 does all of it.  Rows are laid
// out in LDS like the large-tile kernel's (16-byte chunk c of row r at chunk
// c ^ ((r >> 1) & 7)).  Everything the start-up reads is wavefront-uniform and
// comes through the scalar cache, in two round trips.
// ---------------------------------------------------------------------------
constexpr int kStBK = 64, kStRowBytes = kStBK * 2, kStRows = 64, kStUnits = 4, kStBM = 32;
constexpr int kStWBytes = kStRows * kStRowBytes;               // 8 KB of weights per unit
constexpr int kStUnitBytes = kStWBytes + kStBM * kStRowBytes;  // plus 4 KB of tokens
constexpr int kStDmaPerUnit = 3;                               // requests per wavefront and unit

template <typename Mma, bool GATED>
__global__ __launch_bounds__(kThreads, 3) void stream_gemm_kernel(const GemmParams p) {
  using El = typename Mma::El;
  __shared__ __attribute__((aligned(1024))) char smem[kStUnits * kStUnitBytes];
  constexpr int BN_OUT = GATED ? kStRows / 2 : kStRows;
  // Per-XCD ranges of the (block major, n-tile minor) order, cut from the live
  // blocks only: the n-tiles of a block run side by side and share its token
  // rows through one L2 (in the down pass those rows are 1.5 KB x 32 per block
  // and were re-fetched for every n-tile otherwise).
  const int live_mb = (*p.num_post_pad + kStBM - 1) / kStBM;
  const int live = live_mb * p.num_n_tiles;
  const int per_xcd = (live + kXcds - 1) / kXcds;
  const int xslot = blockIdx.x / kXcds;
  const int logical = (blockIdx.x % kXcds) * per_xcd + xslot;
  if (xslot >= per_xcd || logical >= live) return;
  int mb = logical / p.num_n_tiles;
  int nt = logical - mb * p.num_n_tiles;
  {
    // Blocks of one expert (it has more than 32 tokens) stream the same weights.
    // Inside an aligned group of four blocks, reorder a run of g same-expert
    // blocks from (block, n-tile) to (n-tile, block): the g workgroups that
    // read one weight tile then start back to back on one XCD and the second
    // to g-th find the lines in L2 (or already requested).
    const int q0 = mb & ~3;
    int eq[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) eq[i] = q0 + i < live_mb ? p.expert_ids[q0 + i] : -1 - i;
    const int me = mb - q0;
    int lo = me, hi = me;
#pragma unroll
    for (int i = 1; i < 4; ++i) {
      if (lo == me - i + 1 && lo > 0 && eq[lo - 1] == eq[me]) lo = me - i;
      if (hi == me + i - 1 && hi < 3 && eq[hi + 1] == eq[me]) hi = me + i;
    }
    const int g = hi - lo + 1;
    const int li = (me - lo) * p.num_n_tiles + nt;
    nt = li / g;
    mb = q0 + lo + (li - nt * g);
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;
  const int n0 = nt * BN_OUT;

  // second round trip: the expert, and the eight slots whose token rows this wavefront requests
  const int32_t* sid = p.sorted_ids + static_cast<int64_t>(mb) * kStBM;
  const int e = __builtin_amdgcn_readfirstlane(p.expert_ids[mb]);
  const int first = sid[0];
  const int4 s0 = *reinterpret_cast<const int4*>(sid + 8 * wave);
  const int4 s1 = *reinterpret_cast<const int4*>(sid + 8 * wave + 4);
  if (first >= p.numel) return;  // real slots come first: the block is empty
  // What the epilogue needs per slot is fetched now, ahead of the stream: a load
  // issued behind ~100 KB of queued DMA requests would take microseconds to return.
  int tok = p.numel;
  float rw = 1.f;
  if (wave == 0) {
    tok = sid[l32];
    if (p.mul_weight && tok < p.numel) rw = p.topk_w[tok];
  }

  // DMA requests of this wavefront: token rows 8 * wave + lane / 8, weight rows
  // 16 * wave + 8 * j + lane / 8 (j < 2); lane % 8 is the chunk the lane's 16 bytes land in
  const char* a_base = static_cast<const char*>(p.a);
  const char* w_base = static_cast<const char*>(p.w) + static_cast<int64_t>(e) * p.w_stride_e * 2;
  int w_step = kStRowBytes;  // bytes from one K unit to the next
  uint32_t a_off, w_off[2];
  {
    const int q = lane >> 3;
    const int rr = 8 * wave + q;
    int64_t src = mb * kStBM + rr;
    if (!p.a_by_slot) {
      const int lo = (q & 2) ? ((q & 1) ? s0.w : s0.z) : ((q & 1) ? s0.y : s0.x);
      const int hi = (q & 2) ? ((q & 1) ? s1.w : s1.z) : ((q & 1) ? s1.y : s1.x);
      const int tok = (q & 4) ? hi : lo;
      src = tok < p.numel ? tok / p.top_k : 0;
    }
    a_off = static_cast<uint32_t>(src * p.lda * 2 + (((lane & 7) ^ ((rr >> 1) & 7)) << 4));
  }
  if (p.w_tiled) {
    // Weights in 32 KB units of 256 rows (the large-tile kernel's): this workgroup's rows are one
    // or two contiguous pieces of every unit of its n-tile, 32 rows apart from a multiple of 32,
    // so a row's chunks already sit where this kernel's LDS rows want them.
    constexpr int kBigRows = GATED ? 128 : 256;  // output columns covered by one unit
    w_base += static_cast<int64_t>(n0 / kBigRows) * (p.Kd / kStBK) * 32768;
    w_step = 32768;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int rr = 16 * wave + 8 * j + (lane >> 3);
      const int R = GATED ? ((rr >> 5) * 128 + (n0 % kBigRows) + (rr & 31)) : ((n0 % kBigRows) + rr);
      w_off[j] = static_cast<uint32_t>(R * kStRowBytes + ((lane & 7) << 4));
    }
  } else {
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int rr = 16 * wave + 8 * j + (lane >> 3);
    int64_t wrow;
    if constexpr (GATED) {
      const int half = rr >> 5;
      int n = n0 + (rr & 31);
      n = n < p.N ? n : p.N - 1;
      wrow = p.interleaved ? (2 * n + half) : (half * p.N + n);
    } else {
      const int n = n0 + rr;
      wrow = n < p.N ? n : p.N - 1;
    }
    w_off[j] = static_cast<uint32_t>(wrow * p.w_stride_n * 2 + (((lane & 7) ^ ((rr >> 1) & 7)) << 4));
  }
  }
  const uint32_t lds0 = lds_offset_of(smem);
  const uint32_t dma_w = __builtin_amdgcn_readfirstlane(lds0 + 16 * wave * kStRowBytes);
  const uint32_t dma_a = __builtin_amdgcn_readfirstlane(lds0 + kStWBytes + 8 * wave * kStRowBytes);
  auto issue = [&](int u) {
    const uint32_t ring = (u % kStUnits) * kStUnitBytes;
    lds_dma16(a_base + u * kStRowBytes, a_off, dma_a + ring);
#pragma unroll
    for (int j = 0; j < 2; ++j) lds_dma16(w_base + static_cast<int64_t>(u) * w_step, w_off[j], dma_w + ring + j * 1024);
  };

  f32x16 acc0, acc1;
#pragma unroll
  for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
  const int nu = p.Kd / kStBK;
  int rd_k[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) rd_k[kk] = l32 * kStRowBytes + (((2 * kk + lhi) ^ ((l32 >> 1) & 7)) << 4);

  issue(0);
  if (1 < nu) issue(1);
  if (2 < nu) issue(2);
  for (int u = 0; u < nu; ++u) {
    // unit u has landed (only the two younger units may be outstanding) and
    // wavefront 0 is done reading unit u-1, whose ring slot the next request reuses
    if (u + 2 < nu) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * kStDmaPerUnit) : "memory");
    else if (u + 1 < nu) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kStDmaPerUnit) : "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    bare_barrier();
    if (u + 3 < nu) issue(u + 3);
    if (wave == 0) {
      const char* st = smem + (u % kStUnits) * kStUnitBytes;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const uint4 x = *reinterpret_cast<const uint4*>(st + kStWBytes + rd_k[kk]);
        const uint4 w0 = *reinterpret_cast<const uint4*>(st + rd_k[kk]);
        const uint4 w1 = *reinterpret_cast<const uint4*>(st + 32 * kStRowBytes + rd_k[kk]);
        acc0 = Mma::mma(w0, x, acc0);
        acc1 = Mma::mma(w1, x, acc1);
      }
    }
  }

  if (wave != 0) return;
  const int slot = mb * kStBM + l32;
  if (tok < p.numel) {
    const bool fast = n0 + BN_OUT <= p.N && (p.ldc & 3) == 0 && !p.w_scale;
    if constexpr (GATED) {
      if (!fast) store_fragment<El, true>(p, e, acc0, acc1, tok, slot, n0 + 4 * lhi, rw);
      else if (p.activation == MOE_ACT_SILU) stream_store<El, true, MOE_ACT_SILU>(p, e, acc0, acc1, tok, slot, n0 + 4 * lhi, rw);
      else if (p.activation == MOE_ACT_SWIGLUOAI) stream_store<El, true, MOE_ACT_SWIGLUOAI>(p, e, acc0, acc1, tok, slot, n0 + 4 * lhi, rw);
      else stream_store<El, true, MOE_ACT_GELU>(p, e, acc0, acc1, tok, slot, n0 + 4 * lhi, rw);
    } else if (fast) {
      stream_store<El, false, 0>(p, e, acc0, acc0, tok, slot, n0 + 4 * lhi, rw);
      stream_store<El, false, 0>(p, e, acc1, acc1, tok, slot, n0 + 32 + 4 * lhi, rw);
    } else {
      store_fragment<El, false>(p, e, acc0, acc0, tok, slot, n0 + 4 * lhi, rw);
      store_fragment<El, false>(p, e, acc1, acc1, tok, slot, n0 + 32 + 4 * lhi, rw);
    }
  }
}

template <typename Mma, bool GATED>
int launch_stream(GemmParams& p, int64_t sorted_cap, hipStream_t s) {
  p.num_m_blocks = static_cast<int>((sorted_cap + kStBM - 1) / kStBM);
  p.num_n_tiles = (p.N + (GATED ? kStRows / 2 : kStRows) - 1) / (GATED ? kStRows / 2 : kStRows);
  const int64_t tiles = static_cast<int64_t>(p.num_m_blocks) * p.num_n_tiles;
  const int64_t grid = (tiles + kXcds - 1) / kXcds * kXcds;
  if (grid > INT32_MAX) return moe_fail(MOE_ERR_ARG, "fused_experts: grid of %lld workgroups", static_cast<long long>(grid));
  hipLaunchKernelGGL((stream_gemm_kernel<Mma, GATED>), dim3(static_cast<unsigned>(grid)), dim3(kThreads), 0, s, p);
  return moe_check_launch(GATED ? "fused_experts (gate-up pass)" : "fused_experts (down pass)");
}

// Polls a down tile of the one-launch form waits for its m-block's gate-up tiles (about a
// microsecond each): two seconds by default, far beyond any launch of this kernel.
static std::atomic<int> g_wait_limit{2000000};

// Longest m-block range big_plan_kernel may give an XCD: twice the average (a range of
// weight-streaming blocks only, at about half the cost each), never more than all blocks.
static int big_plan_cap(int64_t sorted_cap) {
  const int64_t mbs = (sorted_cap + kBigBM - 1) / kBigBM;
  const int64_t cap = 2 * ((mbs + kXcds - 1) / kXcds);
  return static_cast<int>(cap < mbs ? cap : mbs);
}

template <typename Mma, bool GATED>
int launch_big(GemmParams& p, int64_t sorted_cap, hipStream_t s) {
  constexpr int lds = kBigLdsTotal;
  auto kern = big_gemm_kernel<Mma, GATED>;
  static MoeLdsOptIn opted;  // per instantiation
  if (int rc = moe_opt_in_lds(opted, reinterpret_cast<const void*>(kern), lds, "fused_experts")) return rc;
  p.num_m_blocks = static_cast<int>((sorted_cap + kBigBM - 1) / kBigBM);
  p.num_n_tiles = (p.N + (GATED ? 128 : 256) - 1) / (GATED ? 128 : 256);
  const int64_t tiles = static_cast<int64_t>(p.num_m_blocks) * p.num_n_tiles;
  int64_t grid = (tiles + kXcds - 1) / kXcds * kXcds;
  if (p.xcd_bounds)  // work-balanced ranges: as many slots per XCD as the longest range may have blocks
    grid = static_cast<int64_t>(big_plan_cap(sorted_cap)) * p.num_n_tiles * kXcds;
  if (grid > INT32_MAX) return moe_fail(MOE_ERR_ARG, "fused_experts: grid of %lld workgroups", static_cast<long long>(grid));
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, s, p);
  return moe_check_launch(GATED ? "fused_experts (gate-up pass)" : "fused_experts (down pass)");
}

template <typename Mma, int BM, int BNW, int WAVES_M, bool GATED, bool RAGGED = false>
int launch(const GemmParams& p, hipStream_t s) {
  constexpr int lds = 2 * (BM + BNW) * kRowBytes;
  auto kern = grouped_gemm_kernel<Mma, BM, BNW, WAVES_M, GATED, RAGGED>;
  static MoeLdsOptIn opted;  // per instantiation
  if (int rc = moe_opt_in_lds(opted, reinterpret_cast<const void*>(kern), lds, "fused_experts")) return rc;
  const int64_t tiles = static_cast<int64_t>(p.num_m_blocks) * p.num_n_tiles;
  const int64_t grid = (tiles + kXcds - 1) / kXcds * kXcds;
  if (grid > INT32_MAX) return moe_fail(MOE_ERR_ARG, "fused_experts: grid of %lld workgroups", static_cast<long long>(grid));
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, s, p);
  return moe_check_launch(GATED ? "fused_experts (gate-up pass)" : "fused_experts (down pass)");
}

// Picks the kernel by the caller's alignment block size.  16-bit dtypes: blocks
// of 256 slots go to the large-tile kernel (compute-bound calls), blocks of 32
// slots to the streaming kernel (bandwidth-bound calls).  Everything
// else runs on the register-staged kernels with the largest M tile that
// divides the block size, so that a block is a whole number of tiles of one
// expert.
// The DMA kernels address rows with 32-bit byte offsets from a 64-bit base: both
// operands must span less than 4 GiB (per expert, for the weights).
static bool dma_offsets_fit(const GemmParams& p, bool gated, int64_t sorted_cap, int es) {
  const int64_t a_rows = p.a_by_slot ? sorted_cap : p.numel / p.top_k;
  const int64_t w_rows = gated ? 2LL * p.N : p.N;
  // (16 KB of head room: the per-lane offsets carry up to 8 KB on top of the data's offset)
  const int64_t limit = (1LL << 32) - 16384;
  return a_rows * p.lda * es < limit && w_rows * p.w_stride_n * es < limit;
}

// Whether a 16-bit pass runs on the large-tile kernel.
static bool big_16bit_ok(const GemmParams& p, bool gated, int block_size, int64_t sorted_cap) {
  return block_size % kBigBM == 0 && p.Kd % kBigBK == 0 && dma_offsets_fit(p, gated, sorted_cap, 2);
}

// Gate-up and down pass of the large-tile kernel in one launch (16-bit dtypes).
// p1.xcd_bounds must be set; `done` holds one zeroed counter per m-block.
template <typename Mma>
int launch_big_fused(GemmParams& p1, GemmParams& p2, int block_size, int64_t sorted_cap, int32_t* done,
                     int32_t* status, int down_xcd_shift, hipStream_t s) {
  constexpr int lds = kBigLdsTotal;
  auto kern = big_fused_kernel<Mma>;
  static MoeLdsOptIn opted;
  if (int rc = moe_opt_in_lds(opted, reinterpret_cast<const void*>(kern), lds, "fused_experts")) return rc;
  for (GemmParams* q : {&p1, &p2}) {
    q->align_bs = block_size;
    q->m_major = 1;
    q->num_m_blocks = static_cast<int>((sorted_cap + kBigBM - 1) / kBigBM);
  }
  p1.num_n_tiles = (p1.N + 127) / 128;
  p2.num_n_tiles = (p2.N + 255) / 256;
  // every gate-up tile inside the matrix: its flush takes the 16-byte path, which can write through
  p1.wt_stores = (p1.N % 128 == 0 && p1.ldc % 8 == 0) ? 1 : 0;
  const int cap_mb = big_plan_cap(sorted_cap);
  const int64_t grid = static_cast<int64_t>(cap_mb) * (p1.num_n_tiles + p2.num_n_tiles) * kXcds;
  if (grid > INT32_MAX) return moe_fail(MOE_ERR_ARG, "fused_experts: grid of %lld workgroups", static_cast<long long>(grid));
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, s, p1, p2, done, cap_mb,
                     g_wait_limit.load(std::memory_order_relaxed), status, down_xcd_shift);
  return moe_check_launch("fused_experts (gate-up and down pass, one launch)");
}

template <typename Mma, bool GATED>
int launch_bm(GemmParams& p, int block_size, int64_t sorted_cap, hipStream_t s) {
  p.align_bs = block_size;
  p.m_major = 0;
  const int32_t* bounds = p.xcd_bounds;  // meant for the large-tile kernel only
  p.xcd_bounds = nullptr;
  if constexpr (Mma::kEs != 1) {
    if (p.ragged) {
      // any alignment block is a whole number of 32-slot tiles
      if (block_size % 32 != 0)
        return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: block_size %d is not a multiple of 32", block_size);
      p.num_m_blocks = static_cast<int>((sorted_cap + 31) / 32);
      p.num_n_tiles = (p.N + (GATED ? 128 : 256) - 1) / (GATED ? 128 : 256);
      return launch<Mma, 32, 256, 1, GATED, true>(p, s);
    }
  }
  const bool offsets_fit = dma_offsets_fit(p, GATED, sorted_cap, Mma::kEs);
  if constexpr (Mma::kEs == 1) {
    // a large-tile K step is 128 bytes per row: 128 e4m3 elements
    if (block_size % 256 == 0 && p.Kd % kBigRowBytes == 0 && offsets_fit) {
      p.m_major = 1;
      p.xcd_bounds = bounds;
      return launch_big<MmaE4M3Big<typename Mma::El>, GATED>(p, sorted_cap, s);
    }
  }
  if constexpr (Mma::kEs == 2) {
    if (big_16bit_ok(p, GATED, block_size, sorted_cap)) {
      p.m_major = 1;  // a token block is reused by all its n-tiles through one L2
      p.xcd_bounds = bounds;
      return launch_big<Mma, GATED>(p, sorted_cap, s);
    }
    if (block_size == kStBM && p.Kd % kStBK == 0 && offsets_fit)
      return launch_stream<Mma, GATED>(p, sorted_cap, s);
  }
  if (p.w_tiled)
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: tiled weights run on the large-tile kernel (block_size a multiple "
                    "of 256) and the streaming kernel (block_size 32) only, not with block_size %d", block_size);
  if (block_size % 128 == 0) {
    p.num_m_blocks = static_cast<int>((sorted_cap + 127) / 128);
    p.num_n_tiles = (p.N + (GATED ? 64 : 128) - 1) / (GATED ? 64 : 128);
    return launch<Mma, 128, 128, 2, GATED>(p, s);
  }
  if (block_size % 64 == 0) {
    p.num_m_blocks = static_cast<int>((sorted_cap + 63) / 64);
    p.num_n_tiles = (p.N + (GATED ? 128 : 256) - 1) / (GATED ? 128 : 256);
    return launch<Mma, 64, 256, 1, GATED>(p, s);
  }
  if (block_size % 32 == 0) {
    p.num_m_blocks = static_cast<int>((sorted_cap + 31) / 32);
    p.num_n_tiles = (p.N + (GATED ? 128 : 256) - 1) / (GATED ? 128 : 256);
    return launch<Mma, 32, 256, 1, GATED>(p, s);
  }
  return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: block_size %d is not a multiple of 32", block_size);
}

int elem_size(int dtype) { return dtype == MOE_F32 ? 4 : (dtype == MOE_E4M3 ? 1 : 2); }

// Copies expert weights [E, rows, K] into the unit layout the DMA kernels fetch with plain
// sequential requests.  One workgroup per unit (expert e, n-tile nt, K tile kt): 256 weight rows of
// 128 bytes.  Gated matrices (w13): unit rows [0, 128) are gate rows 128 nt .. + 127, unit rows
// [128, 256) the matching up rows (rows 2n and 2n + 1 when gate and up are interleaved); others
// (w2): rows 256 nt .. + 255.  Inside a unit row r sits at r * 128 and its 16-byte chunk c at chunk
// c ^ ((r >> 1) & 7), the place it has in LDS.
__global__ __launch_bounds__(kThreads) void tile_weights_kernel(const char* __restrict__ src, char* __restrict__ dst,
                                                                int rows, int64_t row_bytes, int n_tiles, int k_tiles,
                                                                int gated, int interleaved) {
  const int64_t unit = blockIdx.x;
  const int kt = static_cast<int>(unit % k_tiles);
  const int nt = static_cast<int>((unit / k_tiles) % n_tiles);
  const int64_t e = unit / k_tiles / n_tiles;
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = (tid >> 3) + 32 * i, pos = tid & 7;
    const int chunk = pos ^ ((r >> 1) & 7);
    int64_t srow;
    if (gated) {
      const int half = r >> 7, n = nt * 128 + (r & 127);
      srow = interleaved ? 2 * n + half : static_cast<int64_t>(half) * (rows / 2) + n;
    } else {
      srow = static_cast<int64_t>(nt) * 256 + r;
    }
    const uint4 v = *reinterpret_cast<const uint4*>(src + (e * rows + srow) * row_bytes + kt * 128 + chunk * 16);
    *reinterpret_cast<uint4*>(dst + unit * kBigUnitBytes + r * 128 + pos * 16) = v;
  }
}

}  // namespace

MOE_EXPORT int moe_tile_expert_weights_supported(int rows, int K, int elem_bytes, int gated) {
  if (rows < 1 || K < 1 || (elem_bytes != 1 && elem_bytes != 2)) return 0;
  return rows % 256 == 0 && (static_cast<int64_t>(K) * elem_bytes) % 128 == 0 ? 1 : 0;
}

MOE_EXPORT int moe_tile_expert_weights(const void* src, void* dst, int E, int rows, int K, int elem_bytes, int gated,
                                       int interleaved, void* stream) {
  if (!src || !dst || E < 1) return moe_fail(MOE_ERR_ARG, "tile_expert_weights: null pointer or E=%d", E);
  if (!moe_tile_expert_weights_supported(rows, K, elem_bytes, gated))
    return moe_fail(MOE_ERR_UNSUPPORTED, "tile_expert_weights: rows=%d must be a multiple of 256 and K=%d x %d bytes a "
                    "multiple of 128", rows, K, elem_bytes);
  if (src == dst) return moe_fail(MOE_ERR_ARG, "tile_expert_weights: source and destination must differ");
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u)
    return moe_fail(MOE_ERR_ARG, "tile_expert_weights: buffers must be 16-byte aligned");
  const int64_t row_bytes = static_cast<int64_t>(K) * elem_bytes;
  const int n_tiles = rows / 256, k_tiles = static_cast<int>(row_bytes / 128);
  const int64_t units = static_cast<int64_t>(E) * n_tiles * k_tiles;
  if (units > INT32_MAX) return moe_fail(MOE_ERR_ARG, "tile_expert_weights: %lld units", static_cast<long long>(units));
  hipLaunchKernelGGL(tile_weights_kernel, dim3(static_cast<unsigned>(units)), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const char*>(src), static_cast<char*>(dst), rows,
                     row_bytes, n_tiles, k_tiles, gated ? 1 : 0, interleaved ? 1 : 0);
  return moe_check_launch("tile_expert_weights");
}

MOE_EXPORT int moe_preferred_block_size(int M, int E, int K, int act_dtype, int weight_dtype) {
  if (E < 1) return 64;
  const int64_t avg = static_cast<int64_t>(M) * K / E;  // routed rows per expert
  if (act_dtype == MOE_F32) {  // register-staged kernels only: the M tile follows the load
    if (avg >= 256) return 256;
    if (avg >= 96) return 128;
    if (avg >= 24) return 64;
    return 32;
  }
  // 16-bit activations: the large-tile kernel, whose two passes go out as one launch,
  // or the streaming kernel with 32-slot blocks.  Padding fragments of a 256-slot block
  // cost neither loads nor MFMAs, so the large tile wins from 16 routed rows per expert
  // on (Qwen3-30B-A3B layer: 0.171 against 0.184 ms at 256 tokens, 0.210 against 0.235 ms
  // at 512; at 192 tokens the streaming kernel still leads, 0.171 against 0.189 ms).
  // e4m3 weights quantise the intermediate between the passes (two launches): from 32
  // rows per expert on (0.181 against 0.193 ms at 512 tokens; 0.172 against 0.166 at 384).
  if (avg >= (weight_dtype == MOE_E4M3 ? 32 : 16)) return 256;
  return 32;
}

MOE_EXPORT int64_t moe_fused_experts_workspace_bytes(int T, int H, int I, int E, int K,
                                                     int block_size, int act_dtype,
                                                     int weight_dtype) {
  if (T < 0 || H < 1 || I < 1 || E < 1 || K < 1 || block_size < 1) return 0;
  const int64_t numel = static_cast<int64_t>(T) * K;
  const int64_t sorted_cap = numel + static_cast<int64_t>(E) * (block_size - 1);
  const int64_t rows = moe_align_up(sorted_cap, block_size);
  const int64_t es = elem_size(act_dtype);
  int64_t bytes = moe_align_up(rows * I * es, 256) + moe_align_up(numel * H * es, 256);
  if (weight_dtype == MOE_E4M3)  // e4m3 copies of x and of the intermediate, one fp32 scale per row
    bytes += moe_align_up(static_cast<int64_t>(T) * H, 256) + moe_align_up(static_cast<int64_t>(T) * 4, 256) +
             moe_align_up(rows * I, 256) + moe_align_up(rows * 4, 256);
  // one counter per 256-slot block (one-launch form of the large-tile passes), then
  // the per-XCD m-block ranges of the large-tile kernel
  return bytes + moe_align_up((sorted_cap + kBigBM - 1) / kBigBM * 4, 256) + 256;
}

// Where in the workspace of a moe_fused_experts call of these sizes the per-XCD ranges (9
// int32) and the per-block counters sit, for moe_align_block_size_planned.  Returns 1 when
// such a call uses them (blocks that are multiples of 256 slots, 16-bit activations), else 0.
MOE_EXPORT int moe_fused_experts_plan_layout(int T, int H, int I, int E, int K, int block_size,
                                             int act_dtype, int weight_dtype, int64_t* bounds_offset,
                                             int64_t* done_offset, int32_t* num_done, int32_t* cap_mb) {
  if (T < 1 || block_size % kBigBM != 0 || act_dtype == MOE_F32) return 0;
  const int64_t need_ws = moe_fused_experts_workspace_bytes(T, H, I, E, K, block_size, act_dtype, weight_dtype);
  if (need_ws <= 0) return 0;
  const int64_t sorted_cap = static_cast<int64_t>(T) * K + static_cast<int64_t>(E) * (block_size - 1);
  const int64_t nd = (sorted_cap + kBigBM - 1) / kBigBM;
  *bounds_offset = need_ws - 256;
  *done_offset = need_ws - 256 - moe_align_up(nd * 4, 256);
  *num_done = static_cast<int32_t>(nd);
  *cap_mb = big_plan_cap(sorted_cap);
  return 1;
}

// Argument checks shared by moe_fused_experts and moe_fused_experts_status.  `cap` receives the
// length of sorted_token_ids the call works with: numel + E * (block_size - 1), which no
// alignment of T * K ids over E experts can exceed.  A longer buffer is accepted and its
// surplus ignored: every region of the workspace is laid out from `cap`, never from the
// caller's figure.
// Whether a 16-bit or fp32 call has rows that are not whole, aligned 16-byte chunks: H or I, a
// weight stride (the expert stride of a single expert carries no meaning) or a base address.
static bool fused_args_ragged(const MoeFusedExpertsArgs* a) {
  if (a->weight_dtype == MOE_E4M3) return false;
  const int chunk = a->act_dtype == MOE_F32 ? 4 : 8;
  if (a->H % chunk || a->I % chunk || a->w13_stride_n % chunk || a->w2_stride_n % chunk) return true;
  if (a->E > 1 && (a->w13_stride_e % chunk || a->w2_stride_e % chunk)) return true;
  return ((reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->w13) |
           reinterpret_cast<uintptr_t>(a->w2) | reinterpret_cast<uintptr_t>(a->out)) & 15u) != 0;
}

static int check_fused_args(const MoeFusedExpertsArgs* a, int64_t* cap, int64_t* need_ws) {
  if (!a) return moe_fail(MOE_ERR_ARG, "fused_experts: null argument block");
  if (a->T < 0 || a->H < 1 || a->I < 1 || a->E < 1 || a->K < 1 || a->block_size < 1)
    return moe_fail(MOE_ERR_ARG, "fused_experts: bad sizes T=%d H=%d I=%d E=%d K=%d block_size=%d", a->T, a->H, a->I,
                    a->E, a->K, a->block_size);
  if (a->T == 0) { *cap = 0; *need_ws = 0; return MOE_OK; }
  if (!a->x || !a->out || !a->w13 || !a->w2 || !a->topk_weights || !a->sorted_token_ids ||
      !a->expert_ids || !a->num_tokens_post_pad)
    return moe_fail(MOE_ERR_ARG, "fused_experts: null tensor pointer");
  if (a->act_dtype != MOE_BF16 && a->act_dtype != MOE_F16 && a->act_dtype != MOE_F32)
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: activation dtype code %d", a->act_dtype);
  if (a->act_dtype == MOE_F32 && a->weight_dtype == MOE_E4M3)
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: e4m3 weights need bf16 or fp16 activations");
  const bool fp8 = a->weight_dtype == MOE_E4M3;
  if (!fp8 && a->weight_dtype != a->act_dtype)
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: weight dtype code %d with activation dtype code %d", a->weight_dtype, a->act_dtype);
  if (fp8 && (!a->w13_scale || !a->w2_scale))
    return moe_fail(MOE_ERR_ARG, "fused_experts: e4m3 weights need w13_scale and w2_scale");
  if (fp8 && (a->H % 16 || a->I % 16 || a->w13_stride_n % 16 || a->w2_stride_n % 16 || a->w13_stride_e % 16 || a->w2_stride_e % 16))
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: e4m3 path needs H, I and weight strides in multiples of 16");
  if (a->activation < MOE_ACT_SILU || a->activation > MOE_ACT_GELU)
    return moe_fail(MOE_ERR_ARG, "fused_experts: unknown activation code %d", a->activation);
  // Rows normally move in 16-byte chunks (8 elements of 16 bits, 4 of fp32).  Sizes, strides or
  // bases that do not allow that take the element-by-element kernel (fused_args_ragged); e4m3 rows
  // are always whole chunks (checked above), and so are their bases:
  const uintptr_t bases = reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->w13) |
                          reinterpret_cast<uintptr_t>(a->w2) | reinterpret_cast<uintptr_t>(a->out);
  if (fp8 && (bases & 15u)) return moe_fail(MOE_ERR_ARG, "fused_experts: tensors must be 16-byte aligned");
  if (bases & (a->act_dtype == MOE_F32 ? 3u : 1u))
    return moe_fail(MOE_ERR_ARG, "fused_experts: tensors must be aligned to their element size");
  if (a->weight_layout != MOE_WEIGHTS_PLAIN && a->weight_layout != MOE_WEIGHTS_TILED)
    return moe_fail(MOE_ERR_ARG, "fused_experts: unknown weight_layout %d", a->weight_layout);
  if (a->weight_layout == MOE_WEIGHTS_TILED) {
    if (fused_args_ragged(a))
      return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: tiled weights need 16-byte aligned tensors");
    if (fp8 || a->act_dtype == MOE_F32)
      return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: tiled weights are for bf16 and fp16 only");
    if (!moe_tile_expert_weights_supported(2 * a->I, a->H, 2, 1) || !moe_tile_expert_weights_supported(a->H, a->I, 2, 0))
      return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: tiled weights need I a multiple of 128 and H a multiple of 256 "
                      "(I=%d, H=%d)", a->I, a->H);
    if (a->w13_stride_n != a->H || a->w13_stride_e != 2LL * a->I * a->H || a->w2_stride_n != a->I ||
        a->w2_stride_e != static_cast<int64_t>(a->H) * a->I)
      return moe_fail(MOE_ERR_ARG, "fused_experts: tiled weights are contiguous [E, rows, K] buffers");
    if (a->block_size % kBigBM != 0 && a->block_size != kStBM)
      return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: tiled weights need block_size 32 or a multiple of 256, not %d",
                      a->block_size);
  }
  const int64_t numel = static_cast<int64_t>(a->T) * a->K;
  const int64_t need_cap = numel + static_cast<int64_t>(a->E) * (a->block_size - 1);
  if (a->sorted_cap < need_cap)
    return moe_fail(MOE_ERR_ARG, "fused_experts: sorted_token_ids holds %lld, needs %lld",
                    static_cast<long long>(a->sorted_cap), static_cast<long long>(need_cap));
  *need_ws = moe_fused_experts_workspace_bytes(a->T, a->H, a->I, a->E, a->K, a->block_size, a->act_dtype,
                                               a->weight_dtype);
  if (!a->workspace || a->workspace_bytes < *need_ws)
    return moe_fail(MOE_ERR_WORKSPACE, "fused_experts: workspace %lld B, needs %lld B",
                    static_cast<long long>(a->workspace_bytes), static_cast<long long>(*need_ws));
  if (reinterpret_cast<uintptr_t>(a->workspace) & 255u)
    return moe_fail(MOE_ERR_WORKSPACE, "fused_experts: workspace must be 256-byte aligned");
  *cap = need_cap;
  return MOE_OK;
}

// Whether both GEMM passes of this call run on the 16-bit large-tile kernel, which then keeps the
// intermediate as 32 KB units in the workspace (I a multiple of 64 is part of big_16bit_ok).
static bool inter_units_ok(const MoeFusedExpertsArgs* a, int64_t cap) {
  if (a->block_size % kBigBM != 0 || a->act_dtype == MOE_F32 || a->weight_dtype == MOE_E4M3) return false;
  if (fused_args_ragged(a)) return false;
  GemmParams p1{}, p2{};
  p1.numel = p2.numel = static_cast<int>(static_cast<int64_t>(a->T) * a->K);
  p1.top_k = p2.top_k = a->K;
  p1.lda = a->H; p1.Kd = a->H; p1.N = a->I; p1.w_stride_n = a->w13_stride_n; p1.a_by_slot = 0;
  p2.lda = a->I; p2.Kd = a->I; p2.N = a->H; p2.w_stride_n = a->w2_stride_n; p2.a_by_slot = 1;
  return big_16bit_ok(p1, true, a->block_size, cap) && big_16bit_ok(p2, false, a->block_size, cap);
}

// Whether this call enqueues the two GEMM passes as one launch (16-bit dtypes, blocks that are
// multiples of 256 slots, both passes requested, operands within the DMA kernels' 32-bit offsets).
static bool uses_one_launch(const MoeFusedExpertsArgs* a, int64_t cap) {
  if (a->block_size % kBigBM != 0 || a->act_dtype == MOE_F32 || a->weight_dtype == MOE_E4M3) return false;
  const int passes = (a->passes & 7) ? a->passes : (a->passes | 7);
  if ((passes & 3) != 3 || (passes & 8)) return false;
  return inter_units_ok(a, cap);
}

MOE_EXPORT int moe_fused_experts_set_wait_limit(int polls) {
  return g_wait_limit.exchange(polls < 0 ? 0 : polls, std::memory_order_relaxed);
}

MOE_EXPORT int moe_fused_experts_status(const MoeFusedExpertsArgs* a) {
  int64_t cap = 0, need_ws = 0;
  if (int rc = check_fused_args(a, &cap, &need_ws)) return rc;
  if (a->T == 0 || !uses_one_launch(a, cap)) return MOE_OK;
  const int32_t* word = reinterpret_cast<const int32_t*>(static_cast<const char*>(a->workspace) + need_ws - 256) +
                        kBigStatusWord;
  int32_t expired = 0;
  hipStream_t s = static_cast<hipStream_t>(a->stream);
  hipError_t e = hipMemcpyAsync(&expired, word, sizeof(expired), hipMemcpyDeviceToHost, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  if (e != hipSuccess) return moe_fail(MOE_ERR_LAUNCH, "fused_experts_status: %s", hipGetErrorString(e));
  if (expired != 0)
    return moe_fail(MOE_ERR_HANDOFF, "fused_experts: %d down tiles gave up waiting for the gate-up tiles of their "
                    "block and wrote NaN rows (one-launch form; passes bit 8 selects two launches)", expired);
  return MOE_OK;
}

MOE_EXPORT int moe_fused_experts(const MoeFusedExpertsArgs* a) {
  int64_t cap = 0, need_ws = 0;
  if (int rc0 = check_fused_args(a, &cap, &need_ws)) return rc0;
  if (a->T == 0) return MOE_OK;
  const bool fp8 = a->weight_dtype == MOE_E4M3;
  const int64_t numel = static_cast<int64_t>(a->T) * a->K;

  hipStream_t s = static_cast<hipStream_t>(a->stream);
  const int64_t es = elem_size(a->act_dtype);
  const int64_t rows = moe_align_up(cap, a->block_size);
  char* inter = static_cast<char*>(a->workspace);
  char* c3 = inter + moe_align_up(rows * a->I * es, 256);
  char* xq = c3 + moe_align_up(numel * a->H * es, 256);                        // fp8 only from here on
  float* xs = reinterpret_cast<float*>(xq + moe_align_up(static_cast<int64_t>(a->T) * a->H, 256));
  char* iq = reinterpret_cast<char*>(xs) + moe_align_up(static_cast<int64_t>(a->T) * 4, 256);
  float* is = reinterpret_cast<float*>(iq + moe_align_up(rows * a->I, 256));

  GemmParams p{};
  p.sorted_ids = a->sorted_token_ids;
  p.expert_ids = a->expert_ids;
  p.num_post_pad = a->num_tokens_post_pad;
  p.topk_w = a->topk_weights;
  p.numel = static_cast<int>(numel);
  p.sorted_cap = cap;
  p.top_k = a->K;
  p.alpha = a->swiglu_alpha;
  p.limit = a->swiglu_limit;
  p.activation = a->activation;
  p.interleaved = a->activation == MOE_ACT_SWIGLUOAI;
  p.w_tiled = a->weight_layout == MOE_WEIGHTS_TILED ? 1 : 0;
  p.ragged = fused_args_ragged(a) ? 1 : 0;
  const int32_t* plan_bounds = nullptr;
  int32_t* plan_done = nullptr;
  if (a->block_size % kBigBM == 0 && a->act_dtype != MOE_F32) {
    // both passes walk the same m-blocks: one plan for the two launches
    int32_t* bounds = reinterpret_cast<int32_t*>(static_cast<char*>(a->workspace) + need_ws - 256);
    const int num_done = static_cast<int>((cap + kBigBM - 1) / kBigBM);
    plan_done = bounds - moe_align_up(static_cast<int64_t>(num_done) * 4, 256) / 4;
    if (!(a->passes & 16)) {  // bit 16: moe_align_block_size_planned already left the plan here
      hipLaunchKernelGGL(big_plan_kernel, dim3(1), dim3(kPlanThreads), 0, s, a->sorted_token_ids,
                         a->num_tokens_post_pad, static_cast<int>(numel), big_plan_cap(cap), bounds,
                         plan_done, num_done);
      if (int rc0 = moe_check_launch("fused_experts (XCD ranges)")) return rc0;
    }
    plan_bounds = bounds;
  }
  p.xcd_bounds = plan_bounds;
  // pass 1: x . W13^T with the gated activation, rows addressed by slot
  p.a = a->x; p.lda = a->H; p.w = a->w13; p.w_stride_e = a->w13_stride_e; p.w_stride_n = a->w13_stride_n;
  p.bias = a->w13_bias; p.bias_stride_e = 2LL * a->I;
  p.c = inter; p.ldc = a->I; p.Kd = a->H; p.N = a->I; p.a_by_slot = 0;
  p.mul_weight = a->apply_router_weight_on_input ? 1 : 0;
  const int passes = (a->passes & 7) ? a->passes : (a->passes | 7);
  int rc = MOE_OK;
  // When both passes run on the 16-bit large-tile kernel the intermediate lives in the workspace as
  // 32 KB units (256 slots x one K tile of the down pass, LDS order): the gate-up flush writes whole
  // units and the down pass fetches each with plain sequential requests.  The choice depends on the
  // sizes only, never on `passes`, so single passes enqueued apart agree on it.
  const bool inter_tiled = plan_bounds && !fp8 && inter_units_ok(a, cap);
  p.c_tiled = inter_tiled ? 1 : 0;
  if (plan_bounds && !fp8 && !p.ragged && (passes & 3) == 3 && !(passes & 8)) {
    // 16-bit dtypes on the large-tile kernel: both passes in one launch
    GemmParams p2 = p;
    p2.a = inter; p2.lda = a->I; p2.w = a->w2; p2.w_stride_e = a->w2_stride_e; p2.w_stride_n = a->w2_stride_n;
    p2.bias = a->w2_bias; p2.bias_stride_e = a->H;
    p2.c = c3; p2.ldc = a->H; p2.Kd = a->I; p2.N = a->H; p2.a_by_slot = 1;
    p2.mul_weight = a->apply_router_weight_on_input ? 0 : 1;
    p2.c_tiled = 0; p2.a_tiled = inter_tiled ? 1 : 0;
    if (big_16bit_ok(p, true, a->block_size, cap) && big_16bit_ok(p2, false, a->block_size, cap)) {
      int32_t* status = const_cast<int32_t*>(plan_bounds) + kBigStatusWord;
      const int shift = (a->passes & 32) ? 1 : 0;  // test setting: every hand-off crosses XCDs
      rc = a->act_dtype == MOE_BF16 ? launch_big_fused<MmaBF16>(p, p2, a->block_size, cap, plan_done, status, shift, s)
                                    : launch_big_fused<MmaF16>(p, p2, a->block_size, cap, plan_done, status, shift, s);
      if (rc) return rc;
      if (!(passes & 4)) return MOE_OK;
      return moe_sum(a->out, c3, a->T, a->K, a->H, a->act_dtype, a->stream);
    }
  }
  if (fp8 && (passes & 1)) {
    // dynamic per-token e4m3 activations: s[t] = amax|x[t]| / 448
    rc = moe_quant_rows_e4m3(a->x, a->act_dtype, a->T, a->H, reinterpret_cast<uint8_t*>(xq), xs, a->stream);
    if (rc) return rc;
    p.a = xq; p.a_scale = xs; p.w_scale = a->w13_scale; p.w_scale_stride_e = 2LL * a->I;
    rc = a->act_dtype == MOE_BF16 ? launch_bm<MmaE4M3<ElemBF16>, true>(p, a->block_size, cap, s)
                                  : launch_bm<MmaE4M3<ElemF16>, true>(p, a->block_size, cap, s);
  } else if (passes & 1) {
    rc = a->act_dtype == MOE_BF16  ? launch_bm<MmaBF16, true>(p, a->block_size, cap, s)
         : a->act_dtype == MOE_F16 ? launch_bm<MmaF16, true>(p, a->block_size, cap, s)
                                   : launch_bm<MmaF32, true>(p, a->block_size, cap, s);
  }
  if (rc) return rc;

  // pass 2: inter . W2^T times the routed weight, rows written by flat token id
  p.a = inter; p.lda = a->I; p.w = a->w2; p.w_stride_e = a->w2_stride_e; p.w_stride_n = a->w2_stride_n;
  p.bias = a->w2_bias; p.bias_stride_e = a->H;
  p.c = c3; p.ldc = a->H; p.Kd = a->I; p.N = a->H; p.a_by_slot = 1;
  p.mul_weight = a->apply_router_weight_on_input ? 0 : 1;
  p.xcd_bounds = plan_bounds;
  p.c_tiled = 0; p.a_tiled = inter_tiled ? 1 : 0;
  if (fp8 && (passes & 2)) {
    // the activated intermediate is quantised per slot row the same way
    rc = moe_quant_slot_rows_e4m3(inter, a->act_dtype, rows, a->I, reinterpret_cast<uint8_t*>(iq), is,
                                  a->sorted_token_ids, cap, static_cast<int>(numel), a->stream);
    if (rc) return rc;
    p.a = iq; p.a_scale = is; p.w_scale = a->w2_scale; p.w_scale_stride_e = a->H;
    rc = a->act_dtype == MOE_BF16 ? launch_bm<MmaE4M3<ElemBF16>, false>(p, a->block_size, cap, s)
                                  : launch_bm<MmaE4M3<ElemF16>, false>(p, a->block_size, cap, s);
  } else if (passes & 2) {
    rc = a->act_dtype == MOE_BF16  ? launch_bm<MmaBF16, false>(p, a->block_size, cap, s)
         : a->act_dtype == MOE_F16 ? launch_bm<MmaF16, false>(p, a->block_size, cap, s)
                                   : launch_bm<MmaF32, false>(p, a->block_size, cap, s);
  }
  if (rc) return rc;

  // top-k combine (nanovllm/layers/for_moe/moe_easy_kernel.py:26-31)
  if (!(passes & 4)) return MOE_OK;
  return moe_sum(a->out, c3, a->T, a->K, a->H, a->act_dtype, a->stream);
}

