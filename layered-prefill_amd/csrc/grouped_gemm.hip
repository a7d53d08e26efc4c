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
#include "common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

struct MmaBF16 {
  using El = ElemBF16;
  static __device__ __forceinline__ f32x16 mma(const uint4& a, const uint4& b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
struct MmaF16 {
  using El = ElemF16;
  static __device__ __forceinline__ f32x16 mma(const uint4& a, const uint4& b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

struct GemmParams {
  const void* a;        // pass 1: x [T, lda]; pass 2: inter [sorted_cap, lda]
  const void* w;        // [E, rows, Kd], K contiguous
  void* c;              // pass 1: inter [sorted_cap, ldc]; pass 2: c3 [T*K, ldc]
  const void* bias;     // [E, rows] in the activation dtype, or null
  const float* topk_w;  // [T*K]
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
};

constexpr int kThreads = 256;
constexpr int kBK = 64;                  // K elements per LDS tile
constexpr int kRowBytes = kBK * 2;       // 128 B per staged row
constexpr int kXcds = 8;

__device__ __forceinline__ int swizzled(int row, int chunk) {
  return row * kRowBytes + ((chunk ^ ((row >> 1) & 7)) << 4);
}

template <typename Mma, int BM, int BNW, int WAVES_M, bool GATED>
__global__ __launch_bounds__(kThreads) void grouped_gemm_kernel(const GemmParams p) {
  using El = typename Mma::El;
  using S = typename El::S;
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
  const int per_xcd = gridDim.x / kXcds;
  const int logical = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
  if (logical >= p.num_m_blocks * p.num_n_tiles) return;
  const int nt = logical / p.num_m_blocks;
  const int mb = logical - nt * p.num_m_blocks;
  if (mb * BM >= *p.num_post_pad) return;
  const int e = p.expert_ids[mb];
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
    a_src[j] = static_cast<const char*>(p.a) + (src * p.lda + ld_c * 8) * 2;
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
               (static_cast<int64_t>(e) * p.w_stride_e + wrow * p.w_stride_n + ld_c * 8) * 2;
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
  const int nk = (p.Kd + kBK - 1) / kBK;

  auto gload = [&](int kt) {
    const bool in_k = kt * kBK + ld_c * 8 < p.Kd;
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
  S* cbase = static_cast<S*>(p.c);
  const S* bias = static_cast<const S*>(p.bias);
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    const int slot = mb * BM + wm * TM + fm * 32 + l32;
    const int tok = p.sorted_ids[slot];
    if (tok >= p.numel) continue;  // padding slot
    const float rw = p.mul_weight ? p.topk_w[tok] : 1.f;
    const int64_t crow = p.a_by_slot ? tok : slot;  // pass 2 writes by token, pass 1 by slot
#pragma unroll
    for (int fo = 0; fo < FNO; ++fo) {
      const int ncol0 = n0 + (GATED ? wn * (TNW / 2) : wn * TNW) + fo * 32 + 4 * lhi;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = ncol0 + 8 * g;
        S o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int col = (n + i < p.N) ? n + i : p.N - 1;
          if constexpr (GATED) {
            float gv = acc[fo][fm][4 * g + i], uv = acc[fo + FNO][fm][4 * g + i];
            if (bias) {
              const int64_t grow = p.interleaved ? 2 * col : col;
              const int64_t urow = p.interleaved ? 2 * col + 1 : p.N + col;
              gv += El::ld(bias[e * p.bias_stride_e + grow]);
              uv += El::ld(bias[e * p.bias_stride_e + urow]);
            }
            if (p.mul_weight) { gv *= rw; uv *= rw; }
            gv = El::ld(El::st(gv));  // the reference stores GEMM1's result in T
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
            float v = acc[fo][fm][4 * g + i];
            if (bias) v += El::ld(bias[e * p.bias_stride_e + col]);
            o[i] = El::st(v * rw);
          }
        }
        S* dst = cbase + crow * p.ldc + n;
        if (n + 3 < p.N && (p.ldc & 3) == 0) {
          *reinterpret_cast<uint2*>(dst) = uint2{static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16),
                                                 static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16)};
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < p.N) dst[i] = o[i];
        }
      }
    }
  }
}

template <typename Mma, int BM, int BNW, int WAVES_M, bool GATED>
int launch(const GemmParams& p, hipStream_t s) {
  constexpr int lds = 2 * (BM + BNW) * kRowBytes;
  auto kern = grouped_gemm_kernel<Mma, BM, BNW, WAVES_M, GATED>;
  static bool attr_set = false;  // per instantiation; dynamic LDS above 64 KB must be opted into
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess)
      return moe_fail(MOE_ERR_LAUNCH, "fused_experts: cannot reserve %d B of LDS: %s", lds, hipGetErrorString(e));
    attr_set = true;
  }
  const int64_t tiles = static_cast<int64_t>(p.num_m_blocks) * p.num_n_tiles;
  const int64_t grid = (tiles + kXcds - 1) / kXcds * kXcds;
  if (grid > INT32_MAX) return moe_fail(MOE_ERR_ARG, "fused_experts: grid of %lld workgroups", static_cast<long long>(grid));
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, s, p);
  return moe_check_launch(GATED ? "fused_experts (gate-up pass)" : "fused_experts (down pass)");
}

template <typename Mma, bool GATED>
int launch_bm(GemmParams& p, int block_size, int64_t sorted_cap, hipStream_t s) {
  p.num_m_blocks = static_cast<int>((sorted_cap + block_size - 1) / block_size);
  switch (block_size) {
    case 128:
      p.num_n_tiles = (p.N + (GATED ? 64 : 128) - 1) / (GATED ? 64 : 128);
      return launch<Mma, 128, 128, 2, GATED>(p, s);
    case 64:
      p.num_n_tiles = (p.N + (GATED ? 128 : 256) - 1) / (GATED ? 128 : 256);
      return launch<Mma, 64, 256, 1, GATED>(p, s);
    case 32:
      p.num_n_tiles = (p.N + (GATED ? 128 : 256) - 1) / (GATED ? 128 : 256);
      return launch<Mma, 32, 256, 1, GATED>(p, s);
    default:
      return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: block_size %d (supported: 32, 64, 128)", block_size);
  }
}

int elem_size(int dtype) { return dtype == MOE_F32 ? 4 : (dtype == MOE_E4M3 ? 1 : 2); }

}  // namespace

MOE_EXPORT int moe_preferred_block_size(int M, int E, int K, int act_dtype, int weight_dtype) {
  (void)act_dtype;
  (void)weight_dtype;
  if (E < 1) return 64;
  const int64_t avg = static_cast<int64_t>(M) * K / E;  // routed rows per expert
  if (avg >= 96) return 128;
  if (avg >= 24) return 64;
  return 32;
}

MOE_EXPORT int64_t moe_fused_experts_workspace_bytes(int T, int H, int I, int E, int K,
                                                     int block_size, int act_dtype,
                                                     int weight_dtype) {
  (void)weight_dtype;
  if (T < 0 || H < 1 || I < 1 || E < 1 || K < 1 || block_size < 1) return 0;
  const int64_t numel = static_cast<int64_t>(T) * K;
  const int64_t sorted_cap = numel + static_cast<int64_t>(E) * (block_size - 1);
  const int64_t rows = moe_align_up(sorted_cap, block_size);
  const int64_t es = elem_size(act_dtype);
  return moe_align_up(rows * I * es, 256) + moe_align_up(numel * H * es, 256);
}

MOE_EXPORT int moe_fused_experts(const MoeFusedExpertsArgs* a) {
  if (!a) return moe_fail(MOE_ERR_ARG, "fused_experts: null argument block");
  if (a->T < 0 || a->H < 1 || a->I < 1 || a->E < 1 || a->K < 1)
    return moe_fail(MOE_ERR_ARG, "fused_experts: bad sizes T=%d H=%d I=%d E=%d K=%d", a->T, a->H, a->I, a->E, a->K);
  if (a->T == 0) return MOE_OK;
  if (!a->x || !a->out || !a->w13 || !a->w2 || !a->topk_weights || !a->sorted_token_ids ||
      !a->expert_ids || !a->num_tokens_post_pad)
    return moe_fail(MOE_ERR_ARG, "fused_experts: null tensor pointer");
  if (a->act_dtype != MOE_BF16 && a->act_dtype != MOE_F16)
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: activation dtype code %d (bf16 and fp16 are built)", a->act_dtype);
  if (a->weight_dtype != a->act_dtype)
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: weight dtype code %d with activation dtype code %d", a->weight_dtype, a->act_dtype);
  if (a->activation < MOE_ACT_SILU || a->activation > MOE_ACT_GELU)
    return moe_fail(MOE_ERR_ARG, "fused_experts: unknown activation code %d", a->activation);
  if (a->H % 8 || a->I % 8)
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: H=%d and I=%d must be multiples of 8", a->H, a->I);
  if (a->w13_stride_n % 8 || a->w13_stride_e % 8 || a->w2_stride_n % 8 || a->w2_stride_e % 8)
    return moe_fail(MOE_ERR_UNSUPPORTED, "fused_experts: weight strides must be multiples of 8 elements");
  if ((reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->w13) |
       reinterpret_cast<uintptr_t>(a->w2) | reinterpret_cast<uintptr_t>(a->out)) & 15u)
    return moe_fail(MOE_ERR_ARG, "fused_experts: tensors must be 16-byte aligned");
  const int64_t numel = static_cast<int64_t>(a->T) * a->K;
  const int64_t need_cap = numel + static_cast<int64_t>(a->E) * (a->block_size - 1);
  if (a->sorted_cap < need_cap)
    return moe_fail(MOE_ERR_ARG, "fused_experts: sorted_token_ids holds %lld, needs %lld",
                    static_cast<long long>(a->sorted_cap), static_cast<long long>(need_cap));
  const int64_t need_ws = moe_fused_experts_workspace_bytes(a->T, a->H, a->I, a->E, a->K, a->block_size,
                                                            a->act_dtype, a->weight_dtype);
  if (!a->workspace || a->workspace_bytes < need_ws)
    return moe_fail(MOE_ERR_WORKSPACE, "fused_experts: workspace %lld B, needs %lld B",
                    static_cast<long long>(a->workspace_bytes), static_cast<long long>(need_ws));
  if (reinterpret_cast<uintptr_t>(a->workspace) & 255u)
    return moe_fail(MOE_ERR_WORKSPACE, "fused_experts: workspace must be 256-byte aligned");

  hipStream_t s = static_cast<hipStream_t>(a->stream);
  const int64_t es = elem_size(a->act_dtype);
  const int64_t rows = moe_align_up(a->sorted_cap, a->block_size);
  char* inter = static_cast<char*>(a->workspace);
  char* c3 = inter + moe_align_up(rows * a->I * es, 256);

  GemmParams p{};
  p.sorted_ids = a->sorted_token_ids;
  p.expert_ids = a->expert_ids;
  p.num_post_pad = a->num_tokens_post_pad;
  p.topk_w = a->topk_weights;
  p.numel = static_cast<int>(numel);
  p.top_k = a->K;
  p.alpha = a->swiglu_alpha;
  p.limit = a->swiglu_limit;
  p.activation = a->activation;
  p.interleaved = a->activation == MOE_ACT_SWIGLUOAI;

  // pass 1: x . W13^T with the gated activation, rows addressed by slot
  p.a = a->x; p.lda = a->H; p.w = a->w13; p.w_stride_e = a->w13_stride_e; p.w_stride_n = a->w13_stride_n;
  p.bias = a->w13_bias; p.bias_stride_e = 2LL * a->I;
  p.c = inter; p.ldc = a->I; p.Kd = a->H; p.N = a->I; p.a_by_slot = 0;
  p.mul_weight = a->apply_router_weight_on_input ? 1 : 0;
  const int passes = a->passes ? a->passes : 7;
  int rc = MOE_OK;
  if (passes & 1)
    rc = a->act_dtype == MOE_BF16 ? launch_bm<MmaBF16, true>(p, a->block_size, a->sorted_cap, s)
                                  : launch_bm<MmaF16, true>(p, a->block_size, a->sorted_cap, s);
  if (rc) return rc;

  // pass 2: inter . W2^T times the routed weight, rows written by flat token id
  p.a = inter; p.lda = a->I; p.w = a->w2; p.w_stride_e = a->w2_stride_e; p.w_stride_n = a->w2_stride_n;
  p.bias = a->w2_bias; p.bias_stride_e = a->H;
  p.c = c3; p.ldc = a->H; p.Kd = a->I; p.N = a->H; p.a_by_slot = 1;
  p.mul_weight = a->apply_router_weight_on_input ? 0 : 1;
  if (passes & 2)
    rc = a->act_dtype == MOE_BF16 ? launch_bm<MmaBF16, false>(p, a->block_size, a->sorted_cap, s)
                                  : launch_bm<MmaF16, false>(p, a->block_size, a->sorted_cap, s);
  if (rc) return rc;

  // top-k combine (nanovllm/layers/for_moe/moe_easy_kernel.py:26-31)
  if (!(passes & 4)) return MOE_OK;
  return moe_sum(a->out, c3, a->T, a->K, a->H, a->act_dtype, a->stream);
}
