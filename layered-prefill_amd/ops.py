"""Native ops with the signatures of the reference's ``nanovllm.ops`` module
(pybind bindings at csrc/ops.cpp:29-60,97-133 of the reference): out-parameter
style, nothing returned, work enqueued on torch's current stream.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from ._lib import check, lib, require_gpu_tensor, stream_ptr

def _align_workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    """Scratch for the three-launch alignment path, taken from torch's caching
    allocator on every call: the block is tied to the current stream, which is
    the stream the kernels are enqueued on, so its reuse after the call is
    ordered behind them and nothing outlives the call."""
    return torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)


def topk_softmax(topk_weights: torch.Tensor, topk_indices: torch.Tensor,
                 token_expert_indices: torch.Tensor, gating_output: torch.Tensor,
                 renormalize: bool = False) -> None:
    """csrc/moe_topk_softmax_kernels.cu:476-503.  ``renormalize`` (not in the
    reference op; default off) folds nanovllm/layers/for_moe/fused_moe.py:417-418
    into the same launch."""
    require_gpu_tensor(gating_output, "gating_output")
    if gating_output.dtype != torch.float32:
        raise RuntimeError(f"expected scalar type Float but found {gating_output.dtype}")
    if topk_weights.dtype != torch.float32:
        raise RuntimeError(f"expected scalar type Float but found {topk_weights.dtype}")
    if topk_indices.dtype != torch.int32 or token_expert_indices.dtype != torch.int32:
        raise RuntimeError("expected scalar type Int for topk_indices / token_expert_indices")
    for name, t in (("topk_weights", topk_weights), ("topk_indices", topk_indices),
                    ("token_expert_indices", token_expert_indices),
                    ("gating_output", gating_output)):
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
    E = gating_output.size(-1)
    T = gating_output.numel() // E if E else 0
    K = topk_weights.size(-1)
    if topk_weights.numel() != T * K or topk_indices.numel() != T * K \
            or token_expert_indices.numel() != T * K:
        raise RuntimeError("topk_softmax: output tensors must hold num_tokens * topk elements")
    with torch.cuda.device(gating_output.device):
        check(lib().moe_topk_softmax(gating_output.data_ptr(), topk_weights.data_ptr(),
                                     topk_indices.data_ptr(), token_expert_indices.data_ptr(),
                                     T, E, K, int(renormalize), stream_ptr(gating_output.device)))


def gate_topk_softmax_supported(hidden_states: torch.Tensor, gate_weight: torch.Tensor) -> bool:
    """Shapes and dtypes the fused gate + routing kernel takes."""
    return (hidden_states.dtype in (torch.bfloat16, torch.float16)
            and gate_weight.dtype == hidden_states.dtype
            and gate_weight.size(0) in (32, 64, 128) and hidden_states.size(-1) % 64 == 0
            and hidden_states.is_contiguous() and gate_weight.is_contiguous())


def gate_topk_softmax(topk_weights: torch.Tensor, topk_indices: torch.Tensor,
                      token_expert_indices: torch.Tensor, hidden_states: torch.Tensor,
                      gate_weight: torch.Tensor, renormalize: bool = False,
                      logits_out: Optional[torch.Tensor] = None) -> None:
    """Router gate (``x @ gate_weight.T`` in the activation dtype,
    nanovllm/models/qwen3_moe.py:93-104,113) and ``topk_softmax`` in one launch.
    No such op in the reference; out-parameter style as ``topk_softmax``."""
    require_gpu_tensor(hidden_states, "hidden_states")
    require_gpu_tensor(gate_weight, "gate_weight")
    if hidden_states.dtype not in _lib.DTYPE_CODE or gate_weight.dtype != hidden_states.dtype:
        raise RuntimeError(f"gate_topk_softmax: dtypes {hidden_states.dtype} / {gate_weight.dtype}")
    if topk_weights.dtype != torch.float32:
        raise RuntimeError(f"expected scalar type Float but found {topk_weights.dtype}")
    if topk_indices.dtype != torch.int32 or token_expert_indices.dtype != torch.int32:
        raise RuntimeError("expected scalar type Int for topk_indices / token_expert_indices")
    for name, t in (("topk_weights", topk_weights), ("topk_indices", topk_indices),
                    ("token_expert_indices", token_expert_indices),
                    ("hidden_states", hidden_states), ("gate_weight", gate_weight)):
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
    T, H = hidden_states.shape
    E = gate_weight.size(0)
    K = topk_weights.size(-1)
    if gate_weight.size(1) != H:
        raise RuntimeError("gate_topk_softmax: gate_weight must be [num_experts, hidden_size]")
    if topk_weights.numel() != T * K or topk_indices.numel() != T * K \
            or token_expert_indices.numel() != T * K:
        raise RuntimeError("gate_topk_softmax: output tensors must hold num_tokens * topk elements")
    if logits_out is not None and (logits_out.dtype != torch.float32 or logits_out.numel() != T * E
                                   or not logits_out.is_contiguous()):
        raise RuntimeError("gate_topk_softmax: logits_out must be contiguous fp32 [num_tokens, num_experts]")
    with torch.cuda.device(hidden_states.device):
        check(lib().moe_gate_topk_softmax(
            hidden_states.data_ptr(), gate_weight.data_ptr(), _lib.DTYPE_CODE[hidden_states.dtype],
            logits_out.data_ptr() if logits_out is not None else None, topk_weights.data_ptr(),
            topk_indices.data_ptr(), token_expert_indices.data_ptr(), T, H, E, K,
            int(renormalize), stream_ptr(hidden_states.device)))


def moe_align_block_size(topk_ids: torch.Tensor, num_experts: int, block_size: int,
                         sorted_token_ids: torch.Tensor, experts_ids: torch.Tensor,
                         num_tokens_post_pad: torch.Tensor) -> None:
    """csrc/moe_align_block_size_kernels.cu:239-291."""
    align_block_size_planned(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                             num_tokens_post_pad, None)


def moe_align_block_size_static(topk_ids: torch.Tensor, num_experts: int, block_size: int,
                                sorted_token_ids: torch.Tensor, experts_ids: torch.Tensor,
                                num_tokens_post_pad: torch.Tensor) -> None:
    """``moe_align_block_size`` through the entry point that allocates nothing
    (``moe_align_block_size_static``): its scratch is a fixed device array inside the
    library, so neither the library nor this wrapper allocates.  For callers that cannot
    allocate; no counterpart in the reference.  Sizes beyond the built-in scratch raise."""
    require_gpu_tensor(topk_ids, "topk_ids")
    if topk_ids.dtype not in _lib.ID_DTYPE_CODE:
        raise RuntimeError(f"moe_align_block_size_kernel not implemented for '{topk_ids.dtype}'")
    for name, t in (("sorted_token_ids", sorted_token_ids), ("experts_ids", experts_ids),
                    ("num_tokens_post_pad", num_tokens_post_pad)):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous int32 tensor")
    if not topk_ids.is_contiguous():
        raise RuntimeError("topk_ids must be contiguous")
    with torch.cuda.device(topk_ids.device):
        check(lib().moe_align_block_size_static(
            topk_ids.data_ptr(), _lib.ID_DTYPE_CODE[topk_ids.dtype], topk_ids.numel(), num_experts,
            block_size, sorted_token_ids.data_ptr(), sorted_token_ids.numel(), experts_ids.data_ptr(),
            experts_ids.numel(), num_tokens_post_pad.data_ptr(), stream_ptr(topk_ids.device)))


def align_block_size_planned(topk_ids: torch.Tensor, num_experts: int, block_size: int,
                             sorted_token_ids: torch.Tensor, experts_ids: torch.Tensor,
                             num_tokens_post_pad: torch.Tensor, plan) -> None:
    """``moe_align_block_size`` with an optional ``plan`` (not in the reference):
    ``(bounds_ptr, done_ptr, num_done, cap_mb)`` inside the workspace of the
    ``moe_fused_experts`` call that follows, for the entry point that also leaves
    the large-tile kernel's per-XCD ranges and cleared counters there."""
    require_gpu_tensor(topk_ids, "topk_ids")
    if topk_ids.dtype not in _lib.ID_DTYPE_CODE:
        raise RuntimeError(f"moe_align_block_size_kernel not implemented for '{topk_ids.dtype}'")
    for name, t in (("sorted_token_ids", sorted_token_ids), ("experts_ids", experts_ids),
                    ("num_tokens_post_pad", num_tokens_post_pad)):
        if t.dtype != torch.int32:
            raise RuntimeError(f"expected scalar type Int but found {t.dtype} for {name}")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
    if not topk_ids.is_contiguous():
        raise RuntimeError("topk_ids must be contiguous")
    numel = topk_ids.numel()
    L = lib()
    ws_bytes = L.moe_align_workspace_bytes(numel, num_experts)
    ws = _align_workspace(ws_bytes, topk_ids.device) if ws_bytes else None
    common = (topk_ids.data_ptr(), _lib.ID_DTYPE_CODE[topk_ids.dtype], numel, num_experts, block_size,
              sorted_token_ids.data_ptr(), sorted_token_ids.numel(), experts_ids.data_ptr(),
              experts_ids.numel(), num_tokens_post_pad.data_ptr(),
              ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
              stream_ptr(topk_ids.device))
    with torch.cuda.device(topk_ids.device):
        if plan is None:
            check(L.moe_align_block_size(*common))
        else:
            check(L.moe_align_block_size_planned(*common, *plan))


def route_align_supported(num_tokens: int, num_experts: int, topk: int) -> bool:
    """Sizes ``route_align_block_size`` takes (at most 32 tokens, a power-of-two number of
    experts up to 256)."""
    return bool(lib().moe_route_align_supported(num_tokens, num_experts, topk))


def route_align_block_size(topk_weights: torch.Tensor, topk_indices: torch.Tensor,
                           token_expert_indices: torch.Tensor, gating_output: torch.Tensor,
                           renormalize: bool, num_experts: int, block_size: int,
                           sorted_token_ids: torch.Tensor, experts_ids: torch.Tensor,
                           num_tokens_post_pad: torch.Tensor, plan=None) -> None:
    """``topk_softmax`` (with the renormalisation of nanovllm/layers/for_moe/fused_moe.py:417-418)
    and ``moe_align_block_size`` on its ids as one launch; ``plan`` as in
    ``align_block_size_planned``.  Same results as the two ops, bit for bit.  No counterpart in the
    reference, which enqueues them one after the other."""
    require_gpu_tensor(gating_output, "gating_output")
    if gating_output.dtype != torch.float32 or topk_weights.dtype != torch.float32:
        raise RuntimeError("route_align_block_size: expected scalar type Float for gating_output / topk_weights")
    for name, t in (("topk_indices", topk_indices), ("token_expert_indices", token_expert_indices),
                    ("sorted_token_ids", sorted_token_ids), ("experts_ids", experts_ids),
                    ("num_tokens_post_pad", num_tokens_post_pad)):
        if t.dtype != torch.int32:
            raise RuntimeError(f"route_align_block_size: {name} must be int32")
    for name, t in (("topk_weights", topk_weights), ("topk_indices", topk_indices),
                    ("token_expert_indices", token_expert_indices), ("gating_output", gating_output),
                    ("sorted_token_ids", sorted_token_ids), ("experts_ids", experts_ids)):
        if not t.is_contiguous():
            raise RuntimeError(f"route_align_block_size: {name} must be contiguous")
    T, E = gating_output.shape
    K = topk_weights.size(-1)
    if E != num_experts or topk_weights.numel() != T * K or topk_indices.numel() != T * K \
            or token_expert_indices.numel() != T * K:
        raise RuntimeError("route_align_block_size: output tensors must hold num_tokens * topk elements "
                           "and gating_output num_experts columns")
    pb, pd, pn, pc = plan if plan is not None else (None, None, 0, 0)
    with torch.cuda.device(gating_output.device):
        check(lib().moe_route_align_block_size(
            gating_output.data_ptr(), topk_weights.data_ptr(), topk_indices.data_ptr(),
            token_expert_indices.data_ptr(), T, E, K, int(renormalize), block_size,
            sorted_token_ids.data_ptr(), sorted_token_ids.numel(), experts_ids.data_ptr(), experts_ids.numel(),
            num_tokens_post_pad.data_ptr(), stream_ptr(gating_output.device), pb, pd, pn, pc))


def _act_args(out: torch.Tensor, input: torch.Tensor):
    require_gpu_tensor(input, "input")
    if input.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"activation kernel not implemented for '{input.dtype}'")
    if out.dtype != input.dtype:
        raise RuntimeError("out and input must have the same dtype")
    if not (out.is_contiguous() and input.is_contiguous()):
        raise RuntimeError("out and input must be contiguous")
    d = input.size(-1) // 2
    rows = input.numel() // (2 * d) if d else 0
    if out.numel() != rows * d:
        raise RuntimeError("out must have shape [..., d] for input [..., 2 * d]")
    return rows, d


def silu_and_mul(out: torch.Tensor, input: torch.Tensor) -> None:
    """csrc/activation_kernels.cu:68-87: out = silu(input[..., :d]) * input[..., d:]."""
    rows, d = _act_args(out, input)
    with torch.cuda.device(input.device):
        check(lib().moe_silu_and_mul(out.data_ptr(), input.data_ptr(), rows, d,
                                     _lib.DTYPE_CODE[input.dtype], stream_ptr(input.device)))


def swigluoai_and_mul(out: torch.Tensor, input: torch.Tensor, alpha: float = 1.702,
                      limit: float = 7.0) -> None:
    """csrc/activation_kernels.cu:89-109 (gate/up interleaved)."""
    rows, d = _act_args(out, input)
    with torch.cuda.device(input.device):
        check(lib().moe_swigluoai_and_mul(out.data_ptr(), input.data_ptr(), rows, d,
                                          _lib.DTYPE_CODE[input.dtype], alpha, limit,
                                          stream_ptr(input.device)))


def moe_sum(input: torch.Tensor, output: torch.Tensor) -> None:
    """nanovllm/layers/for_moe/moe_easy_kernel.py:26-31: output = input.sum(dim=1)."""
    require_gpu_tensor(input, "input")
    if input.dim() != 3 or output.dim() != 2:
        raise RuntimeError("moe_sum: input must be [T, K, H] and output [T, H]")
    T, K, H = input.shape
    if tuple(output.shape) != (T, H) or output.dtype != input.dtype:
        raise RuntimeError("moe_sum: output must be [T, H] of the input dtype")
    if not (input.is_contiguous() and output.is_contiguous()):
        raise RuntimeError("moe_sum: tensors must be contiguous")
    if input.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"moe_sum not implemented for '{input.dtype}'")
    with torch.cuda.device(input.device):
        check(lib().moe_sum(output.data_ptr(), input.data_ptr(), T, K, H,
                            _lib.DTYPE_CODE[input.dtype], stream_ptr(input.device)))


def _norm_call(out, residual, x, weight, eps, name):
    require_gpu_tensor(x, "x")
    if x.dim() != 2:
        raise RuntimeError(f"{name}: only [num_tokens, hidden_size] inputs are supported "
                           "(the per-head form is used by attention, not by the MoE block)")
    if x.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"{name} not implemented for '{x.dtype}'")
    T, H = x.shape
    tensors = [("out", out), ("x", x)] + ([("residual", residual)] if residual is not None else [])
    for nm, t in tensors:
        if tuple(t.shape) != (T, H) or t.dtype != x.dtype or t.device != x.device:
            raise RuntimeError(f"{name}: {nm} must be [{T}, {H}] of dtype {x.dtype} on {x.device}")
        if H > 1 and T > 0 and t.stride(1) != 1:   # (the stride of a one-element or empty dimension says nothing)
            raise RuntimeError(f"{name}: {nm} must be contiguous in its last dimension")
    if tuple(weight.shape) != (H,) or weight.dtype != x.dtype or not weight.is_contiguous():
        raise RuntimeError(f"{name}: weight must be a contiguous [{H}] tensor of dtype {x.dtype}")
    with torch.cuda.device(x.device):
        check(lib().moe_add_rms_norm(out.data_ptr(), out.stride(0),
                                     residual.data_ptr() if residual is not None else None,
                                     residual.stride(0) if residual is not None else 0,
                                     x.data_ptr(), x.stride(0), weight.data_ptr(),
                                     _lib.DTYPE_CODE[x.dtype], T, H, float(eps), stream_ptr(x.device)))


def rms_norm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """csrc/layernorm_kernels.cu:151-176 (2-D case): out = T(T(x * rsqrt(mean(x^2) + eps)) * weight)."""
    _norm_call(out, None, x, weight, eps, "rms_norm")


def add_rms_norm(out: torch.Tensor, residual: torch.Tensor, x: torch.Tensor, weight: torch.Tensor,
                 eps: float) -> None:
    """csrc/layernorm_kernels.cu:205-232 (2-D case): residual += x (rounded to the dtype),
    out = rms_norm(residual).  Argument order as in nanovllm/layers/custom_ops.py:40-41."""
    _norm_call(out, residual, x, weight, eps, "add_rms_norm")


def tile_expert_weights_supported(w: torch.Tensor, gated: bool) -> bool:
    """Whether ``tile_expert_weights`` takes this [E, rows, K] tensor: bf16 / fp16, contiguous, rows
    a multiple of 256 (gate and up halves of 128 each when gated), K a multiple of 64."""
    return bool(w.dim() == 3 and w.dtype in (torch.bfloat16, torch.float16) and w.is_contiguous()
                and lib().moe_tile_expert_weights_supported(w.size(1), w.size(2), w.element_size(), int(gated)))


def tile_expert_weights(w: torch.Tensor, gated: bool, interleaved: bool = False) -> torch.Tensor:
    """[E, rows, K] expert weights -> a new tensor of the same shape and dtype whose bytes are in the
    unit order of ``moe_tile_expert_weights`` (units of 256 rows x 128 bytes of K in the order they
    take in LDS; for ``gated`` w13, 128 gate rows with their 128 up rows).  To be handed to
    ``fused_experts`` with ``weight_layout="tiled"``; element [e, r, k] of the result is *not*
    weight [e, r, k].  No counterpart in the reference (its loader leaves the tensors row-major,
    nanovllm/layers/fused_moe.py:472-658)."""
    require_gpu_tensor(w, "w")
    if not tile_expert_weights_supported(w, gated):
        raise RuntimeError(f"tile_expert_weights: {tuple(w.shape)} {w.dtype} is not tileable: contiguous bf16/fp16 "
                           "[E, rows, K] with rows % 256 == 0 and K % 64 == 0 expected")
    out = torch.empty_like(w)
    with torch.cuda.device(w.device):
        check(lib().moe_tile_expert_weights(w.data_ptr(), out.data_ptr(), w.size(0), w.size(1), w.size(2),
                                            w.element_size(), int(gated), int(interleaved), stream_ptr(w.device)))
    return out


def quant_rows_e4m3(w: torch.Tensor):
    """[..., cols] -> (e4m3fn codes as uint8 of the same shape, fp32 scales [...]):
    per-row s = amax|w| / 448.  No counterpart in the reference."""
    require_gpu_tensor(w, "w")
    if w.dtype not in _lib.DTYPE_CODE or not w.is_contiguous():
        raise RuntimeError("quant_rows_e4m3: contiguous fp32/fp16/bf16 tensor expected")
    cols = w.size(-1)
    rows = w.numel() // cols
    q = torch.empty(w.shape, dtype=torch.uint8, device=w.device)
    s = torch.empty(w.shape[:-1], dtype=torch.float32, device=w.device)
    with torch.cuda.device(w.device):
        check(lib().moe_quant_rows_e4m3(w.data_ptr(), _lib.DTYPE_CODE[w.dtype], rows, cols,
                                        q.data_ptr(), s.data_ptr(), stream_ptr(w.device)))
    return q, s
