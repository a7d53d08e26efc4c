/*
 * C ABI of libmoe_gfx950.so: the fused-MoE expert path for AMD MI355X
 * (gfx950), a drop-in for the native ops and the Triton grouped GEMM behind
 * layered-prefill's `nanovllm.ops` / `nanovllm/layers/for_moe/fused_moe.py`.
 *
 * Conventions
 *  - Every pointer is a device pointer on the current HIP device unless its
 *    name says otherwise.  The library borrows them for the enqueued work
 *    only; it never allocates, frees or retains device memory, never
 *    synchronises the device and never copies device -> host (one exception,
 *    named as such below: moe_fused_experts_status waits for the stream and
 *    reads one word back).  All launch dimensions come from upper bounds known
 *    on the host, so each call can be recorded into a HIP graph.
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *  - Return value 0 = enqueued; negative = rejected, nothing enqueued.
 *    `moe_last_error()` then returns a thread-local, human-readable reason.
 *  - Host-side state: the per-device "large LDS opted in" flags of the kernels, the
 *    wait limit of moe_fused_experts_set_wait_limit and the per-device address of the
 *    built-in scratch array of moe_align_block_size_static, all atomics; entry points
 *    may be called from several host threads.
 *  - Scratch memory comes from the caller (`workspace`), sized by the
 *    matching `*_workspace_bytes` function, 256-byte aligned.
 */
#ifndef MOE_GFX950_H_
#define MOE_GFX950_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes for activations / weights / outputs */
enum MoeDtype { MOE_F32 = 0, MOE_F16 = 1, MOE_BF16 = 2, MOE_E4M3 = 3 };
/* dtype codes for `topk_ids` handed to moe_align_block_size
   (csrc/dispatch_utils.h:16-24 dispatches the same integral types) */
enum MoeIdDtype { MOE_ID_I32 = 0, MOE_ID_I64 = 1, MOE_ID_I16 = 2, MOE_ID_I8 = 3, MOE_ID_U8 = 4 };
enum MoeActivation { MOE_ACT_SILU = 0, MOE_ACT_SWIGLUOAI = 1, MOE_ACT_GELU = 2 };
/* memory layout of the expert weights handed to moe_fused_experts */
enum MoeWeightLayout {
  MOE_WEIGHTS_PLAIN = 0, /* [E, rows, K] row-major, as the reference's loader leaves them       */
  MOE_WEIGHTS_TILED = 1  /* the same bytes re-ordered once by moe_tile_expert_weights            */
};

enum MoeError {
  MOE_OK = 0,
  MOE_ERR_ARG = -1,        /* bad shape / null pointer / unsupported value */
  MOE_ERR_UNSUPPORTED = -2,/* valid request this build has no kernel for    */
  MOE_ERR_WORKSPACE = -3,  /* workspace missing or too small                */
  MOE_ERR_LAUNCH = -4,     /* hipLaunchKernel reported an error             */
  MOE_ERR_HANDOFF = -5     /* moe_fused_experts_status: a bounded device-side wait of the
                              previous call expired; its output holds NaN rows */
};

const char* moe_last_error(void);
/* ABI version of this header; bumped when a signature changes. */
int moe_abi_version(void);

/* Replaces `topk_softmax` (csrc/moe_topk_softmax_kernels.cu:476-503, bound at
 * csrc/ops.cpp:46-51,110-117).  Row-wise fp32 softmax over E experts, then K
 * rounds of argmax with the lower index winning ties.  Writes
 * topk_weights[T,K] (softmax values, or those divided by their sum over k when
 * renormalize != 0, which is nanovllm/layers/for_moe/fused_moe.py:417-418),
 * topk_ids[T,K] and token_expert_indices[T,K] = k*T + row.  Needs no
 * workspace for any E in [1, 16384] (a row beyond 1024 columns is kept in LDS
 * by the one wavefront that owns it; MOE_ERR_UNSUPPORTED above 16384);
 * requires K <= E. */
int moe_topk_softmax(const float* gating_output, float* topk_weights, int32_t* topk_ids,
                     int32_t* token_expert_indices, int T, int E, int K, int renormalize,
                     void* stream);

/* Router gate fused in front of `topk_softmax`: logits = x . gate_weight^T (the
 * `ReplicatedLinear` gate of nanovllm/models/qwen3_moe.py:93-104 followed by the
 * call at :113-118; nanovllm/layers/linear.py:53-60), rounded to the activation
 * dtype as that layer's output is, then the routing of moe_topk_softmax.  The
 * logits stay on chip; `logits_out` ([T, E] fp32, may be NULL) receives them when
 * the caller wants to inspect them.  x [T, H] and gate_weight [E, H] are
 * contiguous bf16 or fp16 (MoeDtype code), 16-byte aligned.  Supported shapes:
 * E in {32, 64, 128}, H a multiple of 64; anything else returns
 * MOE_ERR_UNSUPPORTED and the caller runs the gate and moe_topk_softmax apart. */
int moe_gate_topk_softmax(const void* x, const void* gate_weight, int dtype, float* logits_out,
                          float* topk_weights, int32_t* topk_ids, int32_t* token_expert_indices,
                          int T, int H, int E, int K, int renormalize, void* stream);

/* Replaces `moe_align_block_size` (csrc/moe_align_block_size_kernels.cu:239-291,
 * bound at csrc/ops.cpp:53-60,119-126).  `sorted_token_ids` (capacity
 * sorted_cap >= numel + E*(block_size-1)) receives, per expert in ascending
 * expert order, the flat indices i with topk_ids[i] == e in ascending order,
 * padded to a multiple of block_size with the value numel; every slot past
 * the last segment is numel too.  `expert_ids` (capacity expert_cap >=
 * ceil(sorted_cap/block_size)) names the expert of each block and is 0 past
 * the last used block.  `num_tokens_post_pad[0]` is the padded total.  Ids
 * outside [0, E) are dropped.  E <= 1024.  The stable order is produced
 * without global atomics, so results are deterministic. */
int64_t moe_align_workspace_bytes(int64_t numel, int E);
int moe_align_block_size(const void* topk_ids, int ids_dtype, int64_t numel, int E,
                         int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                         int32_t* expert_ids, int64_t expert_cap, int32_t* num_tokens_post_pad,
                         void* workspace, int64_t workspace_bytes, void* stream);

/* moe_align_block_size without a workspace argument and without any allocation.  No
 * counterpart in the reference; it is for callers that cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  The scratch the
 * large path needs (per-segment histograms, moe_align_workspace_bytes) lives in a 4 MiB
 * device array inside the library, one copy per GPU, held until the process ends; sizes
 * that need more are rejected with MOE_ERR_WORKSPACE (at 128 experts the limit is about
 * 4 million ids, at 1024 experts about 520 thousand).  Every call on a GPU shares that
 * GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls on one
 * stream are ordered and each call overwrites what it reads, so nothing needs clearing.
 * The first call on a device looks the array's address up (hipGetSymbolAddress); make that
 * call outside graph capture.  Results are those of moe_align_block_size, bit for bit. */
int moe_align_block_size_static(const void* topk_ids, int ids_dtype, int64_t numel, int E,
                                int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                                int32_t* expert_ids, int64_t expert_cap,
                                int32_t* num_tokens_post_pad, void* stream);

/* The same alignment for block_size 256, which also leaves in the workspace of the
 * moe_fused_experts call that follows what that call would otherwise compute with a launch
 * of its own: the per-XCD m-block ranges of the large-tile kernel (`plan_bounds`, 9 int32)
 * and its cleared per-block counters (`plan_done`, `plan_num_done` int32); the four values
 * come from moe_fused_experts_plan_layout, and that call is then made with bit 16 of
 * `passes` set.  No counterpart in the reference (its Triton launch needs no plan).
 * moe_align_can_plan says whether the size is served (tables of E x segments in LDS). */
int moe_align_can_plan(int64_t numel, int E);
int moe_align_block_size_planned(const void* topk_ids, int ids_dtype, int64_t numel, int E,
                                 int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                                 int32_t* expert_ids, int64_t expert_cap,
                                 int32_t* num_tokens_post_pad, void* workspace,
                                 int64_t workspace_bytes, void* stream, int32_t* plan_bounds,
                                 int32_t* plan_done, int plan_num_done, int plan_cap_mb);


/* moe_topk_softmax followed by moe_align_block_size (with the plan of
 * moe_align_block_size_planned when `plan_bounds` is not NULL) as ONE launch, for the smallest
 * batches of a decode loop: the reference enqueues these as two ops back to back
 * (nanovllm/layers/fused_moe.py:693-741 then nanovllm/layers/for_moe/fused_moe.py:575-577), each a
 * few microseconds, so every launch saved counts.  Results are those of the two calls, bit for bit:
 * `topk_ids` ([T, K] int32) is what gets aligned.  Served sizes (moe_route_align_supported returns
 * 1): T <= 32 (one workgroup routes the rows: beyond 32 the two kernels, whose router spreads over
 * the chip, are faster), E a power of two <= 256, K <= E; otherwise MOE_ERR_UNSUPPORTED and the
 * caller routes and aligns apart.  No workspace. */
int moe_route_align_supported(int T, int E, int K);
int moe_route_align_block_size(const float* gating_output, float* topk_weights, int32_t* topk_ids,
                               int32_t* token_expert_indices, int T, int E, int K, int renormalize,
                               int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                               int32_t* expert_ids, int64_t expert_cap, int32_t* num_tokens_post_pad,
                               void* stream, int32_t* plan_bounds, int32_t* plan_done, int plan_num_done,
                               int plan_cap_mb);

/* Replaces `silu_and_mul` (csrc/activation_kernels.cu:68-87, bound at
 * csrc/ops.cpp:29-31,99-103): out[r,i] = T(silu(in[r,i])) * in[r,d+i]. */
int moe_silu_and_mul(void* out, const void* in, int64_t rows, int d, int dtype, void* stream);

/* Replaces `swigluoai_and_mul` (csrc/activation_kernels.cu:89-109): gate and
 * up interleaved along the last dimension. */
int moe_swigluoai_and_mul(void* out, const void* in, int64_t rows, int d, int dtype, float alpha,
                          float limit, void* stream);

/* Replaces `add_rms_norm` and `rms_norm` for 2-D inputs (csrc/layernorm_kernels.cu:205-232
 * and :151-176, kernels :77-108 and :10-35, bound at csrc/ops.cpp:16-27,103-109): the norm
 * in front of the MoE block.  residual != NULL: s = x + residual in fp32, residual = T(s),
 * out = T(T(residual * rsqrt(mean(s^2) + eps)) * weight); residual == NULL: the same with
 * s = x and nothing stored back.  Strides are element strides of dimension 0; the last
 * dimension is contiguous.  `out` may be `x`. */
int moe_add_rms_norm(void* out, int64_t out_stride, void* residual, int64_t residual_stride,
                     const void* x, int64_t x_stride, const void* weight, int dtype, int64_t T,
                     int H, float eps, void* stream);

/* Replaces `moe_sum` (nanovllm/layers/for_moe/moe_easy_kernel.py:26-31):
 * out[t,:] = sum_k in[t,k,:], fp32 accumulation, one rounding. */
int moe_sum(void* out, const void* in, int64_t T, int K, int H, int dtype, void* stream);

/* Replaces the body of `fused_experts_impl` after alignment
 * (nanovllm/layers/for_moe/fused_moe.py:579-631): grouped GEMM x*W13^T with the
 * gated activation fused into its epilogue, grouped GEMM with W2^T times the
 * routed weight, and the top-k combine.  `out` may alias `x` (inplace=True at
 * nanovllm/layers/fused_moe.py:203-216).  Any H and I with bf16, fp16 and fp32 weights, as the
 * Triton kernel's K and N masks allow (for_moe/fused_moe.py:191-205,218-223): the tuned kernels
 * move rows in 16-byte chunks, and a call whose H, I or weight strides are not multiples of 16
 * bytes, or whose tensors are only element-aligned, runs both GEMM passes on an
 * element-by-element variant of the register-staged kernel (correct, untuned; plain weight
 * layout only).  e4m3 weights: H, I and strides multiples of 16, tensors 16-byte aligned. */
typedef struct MoeFusedExpertsArgs {
  /* tensors */
  const void* x;             /* [T, H] activations, row-major contiguous            */
  void* out;                 /* [T, H] result, same dtype as x                      */
  const void* w13;           /* [E, 2I, H] gate rows [0,I) then up rows [I,2I); or its
                                tiled form (weight_layout)                          */
  const void* w2;            /* [E, H, I]; or its tiled form                        */
  const void* w13_bias;      /* [E, 2I] or NULL                                     */
  const void* w2_bias;       /* [E, H] or NULL                                      */
  const float* w13_scale;    /* fp8 only: [E, 2I] per-output-channel scales, else NULL */
  const float* w2_scale;     /* fp8 only: [E, H], else NULL                         */
  const float* topk_weights; /* [T, K] fp32                                          */
  const int32_t* sorted_token_ids;    /* from moe_align_block_size                  */
  const int32_t* expert_ids;
  const int32_t* num_tokens_post_pad; /* read on the device only                    */
  void* workspace;           /* intermediates and launch bookkeeping of this call: one call at a
                                time per workspace (two calls in flight need two workspaces) */
  int64_t workspace_bytes;
  /* element strides of the expert dimension and the row dimension of the
     weights (last dimension is contiguous) */
  int64_t w13_stride_e, w13_stride_n, w2_stride_e, w2_stride_n;
  /* sizes */
  int32_t T, H, I, E, K;
  int32_t block_size;        /* the block_size the alignment was made with          */
  int64_t sorted_cap;        /* length of sorted_token_ids, >= T*K + E*(block_size-1); the
                                alignment must have been made with the same E and
                                block_size, so nothing lives beyond that length and a
                                longer buffer's surplus is ignored                   */
  int32_t act_dtype;         /* MoeDtype of x / out / biases                         */
  int32_t weight_dtype;      /* MoeDtype of w13 / w2 (MOE_E4M3 selects the fp8 path) */
  int32_t activation;        /* MoeActivation                                        */
  int32_t apply_router_weight_on_input;
  float swiglu_alpha, swiglu_limit;
  /* bit mask of the passes to enqueue: 1 gate-up GEMM + activation, 2 down GEMM
     times routed weight, 4 top-k combine; 0 means all three.  Lets a profiler
     or benchmark time one pass alone (the later passes then read whatever the
     workspace holds).  Bit 8 keeps the two GEMM passes in separate launches
     where the library would otherwise enqueue them as one.  Bit 16: the
     workspace already holds the plan (moe_align_block_size_planned).  Bit 32 (for
     tests of the one-launch form): its down tiles run on the XCD next to the one
     that ran their block's gate-up tiles, so every hand-off crosses two L2s; the
     result is the same, bit for bit. */
  int32_t passes;
  int32_t weight_layout;     /* MoeWeightLayout of w13 and w2 (both): 0 = plain                   */
  void* stream;
} MoeFusedExpertsArgs;

int64_t moe_fused_experts_workspace_bytes(int T, int H, int I, int E, int K, int block_size,
                                          int act_dtype, int weight_dtype);
int moe_fused_experts(const MoeFusedExpertsArgs* args);

/* No counterpart in the reference (its two Triton launches need no hand-off).  With 16-bit
 * dtypes and blocks of 256 slots moe_fused_experts enqueues both GEMM passes as one launch,
 * in which the down tiles of a 256-slot block wait on the device, for a bounded number of
 * polls, until the gate-up tiles of that block have been counted in.  A down tile whose
 * wait expires does not compute: it fills its rows of the result with NaN (which reach
 * `out` through the top-k combine) and counts itself in a status word of the workspace that
 * the next call's plan clears.  moe_fused_experts_status, given the argument block of the
 * most recent moe_fused_experts call on that workspace, copies the word to the host,
 * WAITS FOR `stream` (the only entry point of this library that synchronises) and returns 0,
 * or MOE_ERR_HANDOFF when waits expired (moe_last_error says how many).  Calls that do not
 * use the one-launch form return 0 without touching the device. */
int moe_fused_experts_status(const MoeFusedExpertsArgs* args);
/* Polls (about a microsecond each) a down tile waits before it gives up; default 2,000,000.
 * Process-wide, read at every moe_fused_experts call; returns the previous value.  0 makes
 * every down tile that finds its block incomplete give up at once: the host-forced error
 * path for tests (all kernels still exit normally). */
int moe_fused_experts_set_wait_limit(int polls);
/* Offsets into the workspace (and sizes) of the plan that moe_align_block_size_planned
 * writes for a moe_fused_experts call of these sizes; returns 1 when the call uses one. */
int moe_fused_experts_plan_layout(int T, int H, int I, int E, int K, int block_size, int act_dtype,
                                  int weight_dtype, int64_t* bounds_offset, int64_t* done_offset,
                                  int32_t* num_done, int32_t* cap_mb);

/* The M-tile (alignment block_size) the grouped GEMMs run best with for M
 * tokens; plays the role of config["BLOCK_SIZE_M"] chosen by
 * try_get_optimal_moe_config (nanovllm/layers/for_moe/fused_moe.py:354-390). */
int moe_preferred_block_size(int M, int E, int K, int act_dtype, int weight_dtype);

/* One-time re-ordering of expert weights for the DMA kernels (no counterpart in the reference, whose
 * loader, nanovllm/layers/fused_moe.py:472-658, leaves `w13_weight [E, 2I, H]` / `w2_weight [E, H, I]`
 * row-major; the layer owns these tensors, nothing else reads them, so the layer may re-order them
 * after loading).  `src` [E, rows, K] contiguous -> `dst`, the same number of bytes, as units of 256
 * weight rows x 128 bytes of K (one unit = what a workgroup stages in LDS per K step), units ordered
 * [expert][rows / 256][K * elem_bytes / 128]; inside a unit the bytes are in the order they take in
 * LDS.  `gated` != 0 (w13): a unit holds 128 gate rows and the 128 matching up rows (`interleaved`
 * != 0: gate row n is source row 2n, up row n is 2n + 1, the swigluoai form).  Every 128-byte piece
 * of a weight row that the kernels fetch then sits next to the pieces fetched with it: one
 * sequential 32 KB read per unit instead of 256 pieces a row stride apart.  Results of
 * moe_fused_experts are bit-identical for both layouts.  rows must be a multiple of 256 and
 * K * elem_bytes a multiple of 128 (moe_tile_expert_weights_supported returns 1); src != dst. */
int moe_tile_expert_weights_supported(int rows, int K, int elem_bytes, int gated);
int moe_tile_expert_weights(const void* src, void* dst, int E, int rows, int K, int elem_bytes, int gated,
                            int interleaved, void* stream);

/* fp8 helpers (no counterpart in the reference, which asserts the scales are
 * None at nanovllm/layers/for_moe/fused_moe.py:248-249): per-output-channel
 * e4m3 quantisation of a [rows, cols] weight matrix, s[r] = amax|w[r,:]|/448. */
int moe_quant_rows_e4m3(const void* w, int src_dtype, int64_t rows, int cols, uint8_t* q,
                        float* scales, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_GFX950_H_ */
