"""Host side of the fused-MoE expert path, mirroring the reference's
``nanovllm/layers/for_moe/fused_moe.py`` (same function names, argument order,
defaults, assertions and return values) on top of libmoe_gfx950.so.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Tuple

import torch

from . import _lib, ops
from ._lib import MoeFusedExpertsArgs, check, lib, stream_ptr


# MOE_CHECK_HANDOFF=1: after every chunk wait for the stream and raise if a bounded device-side
# wait of the one-launch form expired (a debugging aid: it synchronises, so not under graph capture)
_CHECK_HANDOFF = os.environ.get("MOE_CHECK_HANDOFF", "0") == "1"


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int
                         ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """nanovllm/layers/for_moe/fused_moe.py:17-70.  Returns (sorted_token_ids
    [numel + E*(block_size-1)], expert_ids [ceil(that / block_size)],
    num_tokens_post_padded [1]), all int32 on topk_ids' device.  The kernel
    writes every element of all three, so nothing is pre-filled here."""
    return _align_block_size(topk_ids, block_size, num_experts, None)


def _align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int, plan
                      ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``moe_align_block_size``; with ``plan`` (see ``ops.align_block_size_planned``)
    the alignment also prepares the launch of the expert GEMMs that follows."""
    max_num_tokens_padded = topk_ids.numel() + num_experts * (block_size - 1)
    sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=topk_ids.device)
    max_num_m_blocks = cdiv(max_num_tokens_padded, block_size)
    expert_ids = torch.empty((max_num_m_blocks,), dtype=torch.int32, device=topk_ids.device)
    num_tokens_post_pad = torch.empty((1), dtype=torch.int32, device=topk_ids.device)
    ops.align_block_size_planned(topk_ids, num_experts, block_size, sorted_ids, expert_ids,
                                 num_tokens_post_pad, plan)
    return sorted_ids, expert_ids, num_tokens_post_pad


def _route_align_block_size(gating_output: torch.Tensor, renormalize: bool, topk_weights: torch.Tensor,
                            topk_ids: torch.Tensor, block_size: int, num_experts: int, plan
                            ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``fused_topk`` into ``topk_weights`` / ``topk_ids`` and ``moe_align_block_size`` on the
    ids as one launch (``ops.route_align_block_size``)."""
    dev = topk_ids.device
    max_num_tokens_padded = topk_ids.numel() + num_experts * (block_size - 1)
    sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty((cdiv(max_num_tokens_padded, block_size),), dtype=torch.int32, device=dev)
    num_tokens_post_pad = torch.empty((1), dtype=torch.int32, device=dev)
    token_expert_indicies = torch.empty_like(topk_ids)
    ops.route_align_block_size(topk_weights, topk_ids, token_expert_indicies, gating_output, renormalize,
                               num_experts, block_size, sorted_ids, expert_ids, num_tokens_post_pad, plan)
    return sorted_ids, expert_ids, num_tokens_post_pad


def _plan_in_workspace(workspace: torch.Tensor, T: int, H: int, I: int, E: int, K: int, block_size: int,
                       act_code: int, weight_code: int, numel: int):
    """Where the alignment may leave the large-tile kernel's per-XCD ranges and
    cleared counters inside ``workspace`` (the tuple ``ops.align_block_size_planned``
    takes), or None when this call has no use for them."""
    L = lib()
    if block_size != 256 or not L.moe_align_can_plan(numel, E):
        return None
    b_off, d_off = ctypes.c_int64(), ctypes.c_int64()
    n_done, cap_mb = ctypes.c_int32(), ctypes.c_int32()
    if not L.moe_fused_experts_plan_layout(T, H, I, E, K, block_size, act_code, weight_code, ctypes.byref(b_off),
                                           ctypes.byref(d_off), ctypes.byref(n_done), ctypes.byref(cap_mb)):
        return None
    base = workspace.data_ptr()
    return (base + b_off.value, base + d_off.value, n_done.value, cap_mb.value)


def try_get_optimal_moe_config(w1_shape, w2_shape, top_k: int, dtype: Optional[str], M: int,
                               is_marlin: bool = False,
                               block_shape: Optional[list] = None,
                               act_dtype: torch.dtype = torch.bfloat16) -> dict:
    """Role of nanovllm/layers/for_moe/fused_moe.py:354-390.  The reference looks
    up Triton tile tables per device name; the HIP kernels own their tiling, so
    the only entry that still matters to callers is BLOCK_SIZE_M, the block size
    handed to moe_align_block_size.  ``act_dtype`` (not in the reference, whose
    ``dtype`` string only names quantised forms) is the activation dtype: fp32
    runs on other kernels than the 16-bit dtypes and has its own rule."""
    E = w2_shape[0]
    act_code = _lib.DTYPE_CODE[act_dtype]
    weight_code = _lib.E4M3_CODE if dtype == "fp8_w8a8" else act_code
    bm = lib().moe_preferred_block_size(M, E, top_k, act_code, weight_code)
    return {"BLOCK_SIZE_M": bm}


def fused_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int,
               renormalize: bool):
    """nanovllm/layers/for_moe/fused_moe.py:393-419."""
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    M, _ = hidden_states.shape
    topk_weights = torch.empty(M, topk, dtype=torch.float32, device=hidden_states.device)
    topk_ids = torch.empty(M, topk, dtype=torch.int32, device=hidden_states.device)
    token_expert_indicies = torch.empty(M, topk, dtype=torch.int32, device=hidden_states.device)
    gating = gating_output if gating_output.dtype == torch.float32 else gating_output.float()
    ops.topk_softmax(topk_weights, topk_ids, token_expert_indicies, gating.contiguous(),
                     renormalize=renormalize)
    return topk_weights, topk_ids, token_expert_indicies


FUSED_GATE_MIN_TOKENS = 2048


def fused_gate_topk(hidden_states: torch.Tensor, gate_weight: torch.Tensor, topk: int,
                    renormalize: bool):
    """The gate linear (nanovllm/models/qwen3_moe.py:93-104,113) and ``fused_topk``
    (nanovllm/layers/for_moe/fused_moe.py:393-419) as one kernel when the shape
    allows and the batch is large enough for it to pay (a workgroup walks all of
    K for 32 tokens: at a few hundred tokens the library GEMM's wider
    parallelism wins, measured 13 us against 20 us at 256 tokens, 30 us against
    28 us at 8448), else as the two steps the reference runs.  Returns what
    ``fused_topk`` returns."""
    if hidden_states.shape[0] >= FUSED_GATE_MIN_TOKENS and \
            ops.gate_topk_softmax_supported(hidden_states, gate_weight):
        M = hidden_states.shape[0]
        dev = hidden_states.device
        topk_weights = torch.empty(M, topk, dtype=torch.float32, device=dev)
        topk_ids = torch.empty(M, topk, dtype=torch.int32, device=dev)
        token_expert_indicies = torch.empty(M, topk, dtype=torch.int32, device=dev)
        ops.gate_topk_softmax(topk_weights, topk_ids, token_expert_indicies, hidden_states,
                              gate_weight, renormalize=renormalize)
        return topk_weights, topk_ids, token_expert_indicies
    router_logits = torch.nn.functional.linear(hidden_states, gate_weight)
    return fused_topk(hidden_states, router_logits, topk, renormalize)


def fused_experts(hidden_states: torch.Tensor,
                  w1: torch.Tensor,
                  w2: torch.Tensor,
                  w1_bias: Optional[torch.Tensor],
                  w2_bias: Optional[torch.Tensor],
                  topk_weights: torch.Tensor,
                  topk_ids: torch.Tensor,
                  inplace: bool = False,
                  activation: str = "silu",
                  apply_router_weight_on_input: bool = False,
                  per_channel_quant: bool = False,
                  global_num_experts: int = -1,
                  expert_map: Optional[torch.Tensor] = None,
                  w1_scale: Optional[torch.Tensor] = None,
                  w2_scale: Optional[torch.Tensor] = None,
                  w1_zp: Optional[torch.Tensor] = None,
                  w2_zp: Optional[torch.Tensor] = None,
                  a1_scale: Optional[torch.Tensor] = None,
                  a2_scale: Optional[torch.Tensor] = None,
                  block_shape: Optional[list] = None,
                  allow_deep_gemm: bool = False,
                  weight_layout: str = "plain") -> torch.Tensor:
    """nanovllm/layers/for_moe/fused_moe.py:422-460.  ``weight_layout`` (not in the
    reference) is "tiled" when ``w1`` and ``w2`` came out of ``ops.tile_expert_weights``."""
    if inplace:
        fused_experts_impl(hidden_states, w1, w2, topk_weights, topk_ids, True, activation,
                           apply_router_weight_on_input, per_channel_quant, global_num_experts,
                           expert_map, w1_scale, w2_scale, w1_zp, w2_zp, a1_scale, a2_scale,
                           block_shape, w1_bias, w2_bias, weight_layout)
        return hidden_states
    return fused_experts_impl(hidden_states, w1, w2, topk_weights, topk_ids, False, activation,
                              apply_router_weight_on_input, per_channel_quant, global_num_experts,
                              expert_map, w1_scale, w2_scale, w1_zp, w2_zp, a1_scale, a2_scale,
                              block_shape, w1_bias, w2_bias, weight_layout)


def fused_topk_experts(hidden_states: torch.Tensor, gating_output: torch.Tensor, w1: torch.Tensor,
                       w2: torch.Tensor, topk: int, renormalize: bool,
                       w1_bias: Optional[torch.Tensor] = None, w2_bias: Optional[torch.Tensor] = None,
                       inplace: bool = False, activation: str = "silu",
                       apply_router_weight_on_input: bool = False,
                       w1_scale: Optional[torch.Tensor] = None, w2_scale: Optional[torch.Tensor] = None,
                       weight_layout: str = "plain") -> torch.Tensor:
    """``fused_topk`` followed by ``fused_experts``: the two calls of
    ``UnquantizedFusedMoEMethod.apply`` (nanovllm/layers/fused_moe.py:163-216) as one function, so
    that for the smallest batches (``ops.route_align_supported``: up to 32 tokens) routing and
    alignment go out as one launch instead of two.  Same result as the two calls, bit for bit.
    The one launch saves host time (a launch is some 9 us of it), not GPU time: replayed from a HIP
    graph the two kernels take 13.2 us and the one 14.7 us at 32 tokens.  So a call made while the
    stream is being captured enqueues the two kernels."""
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    M, E = gating_output.shape
    if (hidden_states.is_cuda and M > 0 and w1.size(0) == E and ops.route_align_supported(M, E, topk)
            and not torch.cuda.is_current_stream_capturing()):
        gating = gating_output if gating_output.dtype == torch.float32 else gating_output.float()
        topk_weights = torch.empty(M, topk, dtype=torch.float32, device=hidden_states.device)
        topk_ids = torch.empty(M, topk, dtype=torch.int32, device=hidden_states.device)
        out = fused_experts_impl(hidden_states, w1, w2, topk_weights, topk_ids, inplace, activation,
                                 apply_router_weight_on_input, w1_scale is not None, -1, None, w1_scale, w2_scale,
                                 None, None, None, None, None, w1_bias, w2_bias, weight_layout,
                                 _route=(gating.contiguous(), renormalize))
        return hidden_states if inplace else out
    topk_weights, topk_ids, _ = fused_topk(hidden_states, gating_output, topk, renormalize)
    return fused_experts(hidden_states, w1, w2, w1_bias, w2_bias, topk_weights, topk_ids, inplace=inplace,
                         activation=activation, apply_router_weight_on_input=apply_router_weight_on_input,
                         per_channel_quant=w1_scale is not None, w1_scale=w1_scale, w2_scale=w2_scale,
                         weight_layout=weight_layout)


def fused_experts_workspace_bytes(tokens: int, hidden: int, intermediate: int, experts: int,
                                  top_k: int, block_size: int, act_dtype: torch.dtype,
                                  weight_code: Optional[int] = None) -> int:
    act_code = _lib.DTYPE_CODE[act_dtype]
    return lib().moe_fused_experts_workspace_bytes(
        tokens, hidden, intermediate, experts, top_k, block_size, act_code,
        act_code if weight_code is None else weight_code)


def launch_fused_experts(x: torch.Tensor, out: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                         w1_bias: Optional[torch.Tensor], w2_bias: Optional[torch.Tensor],
                         w1_scale: Optional[torch.Tensor], w2_scale: Optional[torch.Tensor],
                         topk_weights: torch.Tensor, sorted_token_ids: torch.Tensor,
                         expert_ids: torch.Tensor, num_tokens_post_padded: torch.Tensor,
                         block_size: int, activation: str = "silu",
                         apply_router_weight_on_input: bool = False,
                         weight_code: Optional[int] = None,
                         workspace: Optional[torch.Tensor] = None, passes: int = 0,
                         weight_layout: str = "plain") -> MoeFusedExpertsArgs:
    """One call of the C entry point ``moe_fused_experts`` on already aligned
    tokens (the part of nanovllm/layers/for_moe/fused_moe.py:579-631 after
    moe_align_block_size).  ``workspace`` (uint8) is allocated when not given;
    ``passes`` selects single passes for profiling (1 gate-up, 2 down, 4
    combine, 0 = all; adding 8 keeps the two GEMM passes in separate launches
    where the library would enqueue them as one).  Returns the argument block
    (what ``fused_experts_status`` takes)."""
    T, H = x.shape
    E, N, _ = w1.shape
    top_k = topk_weights.shape[1]
    act_code = _lib.DTYPE_CODE[x.dtype]
    if weight_code is None:
        weight_code = act_code
    L = lib()
    ws_bytes = L.moe_fused_experts_workspace_bytes(T, H, N // 2, E, top_k, block_size, act_code,
                                                   weight_code)
    if workspace is None:
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    for name, b in (("w1_bias", w1_bias), ("w2_bias", w2_bias)):
        if b is not None:
            assert b.is_contiguous() and b.dtype == x.dtype, f"{name} must be contiguous {x.dtype}"
    args = MoeFusedExpertsArgs(
        x=x.data_ptr(), out=out.data_ptr(), w13=w1.data_ptr(), w2=w2.data_ptr(),
        w13_bias=w1_bias.data_ptr() if w1_bias is not None else None,
        w2_bias=w2_bias.data_ptr() if w2_bias is not None else None,
        w13_scale=w1_scale.data_ptr() if w1_scale is not None else None,
        w2_scale=w2_scale.data_ptr() if w2_scale is not None else None,
        topk_weights=topk_weights.data_ptr(), sorted_token_ids=sorted_token_ids.data_ptr(),
        expert_ids=expert_ids.data_ptr(), num_tokens_post_pad=num_tokens_post_padded.data_ptr(),
        workspace=workspace.data_ptr(), workspace_bytes=workspace.numel(),
        w13_stride_e=w1.stride(0), w13_stride_n=w1.stride(1),
        w2_stride_e=w2.stride(0), w2_stride_n=w2.stride(1),
        T=T, H=H, I=N // 2, E=E, K=top_k, block_size=block_size,
        sorted_cap=sorted_token_ids.numel(), act_dtype=act_code, weight_dtype=weight_code,
        activation=_lib.ACTIVATION_CODE[activation],
        apply_router_weight_on_input=int(apply_router_weight_on_input),
        swiglu_alpha=1.702, swiglu_limit=7.0, passes=passes,
        weight_layout=_lib.WEIGHT_LAYOUT_CODE[weight_layout], stream=stream_ptr(x.device))
    with torch.cuda.device(x.device):
        check(L.moe_fused_experts(args))
    args._keepalive = (workspace,)
    return args


def fused_experts_status(args: MoeFusedExpertsArgs) -> None:
    """``moe_fused_experts_status`` for the argument block of the most recent
    ``launch_fused_experts`` call on its workspace: waits for the stream and raises
    ``RuntimeError`` when a down tile of the one-launch form gave up waiting for
    its block's gate-up tiles (its rows of the result are NaN then).  No
    counterpart in the reference."""
    check(lib().moe_fused_experts_status(args))


def set_wait_limit(polls: int) -> int:
    """``moe_fused_experts_set_wait_limit``: polls a down tile of the one-launch
    form waits before giving up (process-wide); returns the previous value."""
    return lib().moe_fused_experts_set_wait_limit(int(polls))


def quantize_expert_weights(w13: torch.Tensor, w2: torch.Tensor):
    """One-time e4m3 quantisation of expert weights with one scale per output
    channel, s = amax|row| / 448 (no counterpart in the reference).  Returns
    (w13_q, w13_scale, w2_q, w2_scale); the quantised tensors are
    ``torch.float8_e4m3fn`` views."""
    w13_q, w13_s = ops.quant_rows_e4m3(w13.contiguous())
    w2_q, w2_s = ops.quant_rows_e4m3(w2.contiguous())
    return w13_q.view(torch.float8_e4m3fn), w13_s, w2_q.view(torch.float8_e4m3fn), w2_s


_FP8_DTYPES = tuple(getattr(torch, n) for n in ("float8_e4m3fn",) if hasattr(torch, n))


def fused_experts_impl(hidden_states: torch.Tensor,
                       w1: torch.Tensor,
                       w2: torch.Tensor,
                       topk_weights: torch.Tensor,
                       topk_ids: torch.Tensor,
                       inplace: bool = False,
                       activation: str = "silu",
                       apply_router_weight_on_input: bool = False,
                       per_channel_quant: bool = False,
                       global_num_experts: int = -1,
                       expert_map: Optional[torch.Tensor] = None,
                       w1_scale: Optional[torch.Tensor] = None,
                       w2_scale: Optional[torch.Tensor] = None,
                       w1_zp: Optional[torch.Tensor] = None,
                       w2_zp: Optional[torch.Tensor] = None,
                       a1_scale: Optional[torch.Tensor] = None,
                       a2_scale: Optional[torch.Tensor] = None,
                       block_shape: Optional[list] = None,
                       w1_bias: Optional[torch.Tensor] = None,
                       w2_bias: Optional[torch.Tensor] = None,
                       weight_layout: str = "plain", _route=None) -> torch.Tensor:
    """nanovllm/layers/for_moe/fused_moe.py:461-633: align -> gate-up GEMM with
    the gated activation -> down GEMM times the routed weight -> top-k sum, in
    chunks of 64K tokens."""
    # Check constraints (same wording as the reference, :484-493).
    assert hidden_states.size(1) == w1.size(2), (
        f"Hidden size mismatch {hidden_states.size(1)} != {w1.size(2)}")
    assert topk_weights.size() == topk_ids.size(), "topk shape mismatch"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.stride(-1) == 1, "Stride of last dimension must be 1"
    assert w2.stride(-1) == 1, "Stride of last dimension must be 1"
    assert hidden_states.dtype in [torch.float32, torch.float16, torch.bfloat16]
    assert a1_scale is None and a2_scale is None, \
        "static activation scales are not supported (fp8 activations are quantised per token)"
    assert w1_zp is None and w2_zp is None and block_shape is None and expert_map is None
    if activation not in _lib.ACTIVATION_CODE:
        raise ValueError(f"Unsupported FusedMoe activation: {activation}")
    if weight_layout not in _lib.WEIGHT_LAYOUT_CODE:
        raise ValueError(f"Unsupported weight_layout: {weight_layout}")

    fp8 = w1.dtype in _FP8_DTYPES or (w1_scale is not None)
    if fp8:
        # e4m3 weights with one fp32 scale per output channel (w1_scale [E, 2I], w2_scale
        # [E, H]); activations are quantised per token inside the call.  The reference
        # carries these keywords but asserts them None (for_moe/fused_moe.py:248-249).
        assert w1_scale is not None and w2_scale is not None, "fp8 weights need w1_scale and w2_scale"
        assert w1.dtype in _FP8_DTYPES + (torch.uint8,) and w2.dtype == w1.dtype, \
            "fp8 weights must be float8_e4m3fn (or its uint8 codes)"
        assert tuple(w1_scale.shape) == tuple(w1.shape[:2]) and tuple(w2_scale.shape) == tuple(w2.shape[:2]), \
            "per-output-channel scales expected"
        assert w1_scale.dtype == torch.float32 and w2_scale.dtype == torch.float32
        assert w1_scale.is_contiguous() and w2_scale.is_contiguous()
        assert w1_bias is None and w2_bias is None, "biases are not supported on the fp8 path"
        weight_code = _lib.E4M3_CODE
    else:
        assert w1.dtype == hidden_states.dtype and w2.dtype == hidden_states.dtype, \
            "weights and activations must share a dtype"
        weight_code = _lib.DTYPE_CODE[w1.dtype]

    num_tokens = hidden_states.size(0)
    E, N, _ = w1.size()
    K = w2.size(1)
    assert w2.size(2) == N // 2 and w2.size(0) == E, "w2 must be [E, H, I] for w1 [E, 2I, H]"
    if global_num_experts == -1:
        global_num_experts = E
    # without an expert map (rejected above) every expert is local
    assert global_num_experts == E, "global_num_experts must equal the number of local experts (no expert parallelism)"
    # Like the reference's Triton kernel, which masks ragged K and N
    # (for_moe/fused_moe.py:191-205,218-223), any hidden and intermediate size is taken with
    # 16-bit and fp32 weights: rows that are not whole, aligned 16-byte chunks go through an
    # element-by-element kernel.  e4m3 rows are moved in 16-byte chunks only (the reference has
    # no such path):
    if fp8:
        assert hidden_states.size(1) % 16 == 0 and (N // 2) % 16 == 0, \
            "hidden size and intermediate size must be multiples of 16 with e4m3 weights"
        # (the stride of a dimension of size 1 carries no meaning)
        assert all(t.stride(dim) % 16 == 0 for t in (w1, w2) for dim in (0, 1) if t.size(dim) > 1), \
            "weight strides must be multiples of 16 elements with e4m3 weights"
        assert all(t.data_ptr() % 16 == 0 for t in (hidden_states, w1, w2)), "tensors must be 16-byte aligned"
    _lib.require_gpu_tensor(hidden_states, "hidden_states")
    top_k_num = topk_ids.size(1)
    CHUNK_SIZE: int = 64 * 1024
    M = min(num_tokens, CHUNK_SIZE)
    config_dtype = "fp8_w8a8" if fp8 else None
    config = try_get_optimal_moe_config(w1.size(), w2.size(), top_k_num, config_dtype, M,
                                        act_dtype=hidden_states.dtype)

    out_hidden_states = hidden_states if inplace else torch.empty_like(hidden_states)
    if topk_weights.dtype != torch.float32:
        topk_weights = topk_weights.float()
    if topk_ids.dtype != torch.int32:
        topk_ids = topk_ids.to(torch.int32)
    topk_weights = topk_weights.contiguous()
    topk_ids = topk_ids.contiguous()

    L = lib()
    dev = hidden_states.device
    act_code = _lib.DTYPE_CODE[hidden_states.dtype]
    for chunk in range((num_tokens // CHUNK_SIZE) + 1):
        begin, end = chunk * CHUNK_SIZE, min((chunk + 1) * CHUNK_SIZE, num_tokens)
        tokens_in_chunk = end - begin
        if tokens_in_chunk <= 0:
            break
        if tokens_in_chunk < CHUNK_SIZE and chunk > 0:
            config = try_get_optimal_moe_config(w1.size(), w2.size(), top_k_num, config_dtype,
                                                tokens_in_chunk, act_dtype=hidden_states.dtype)
        bm = config["BLOCK_SIZE_M"]
        curr_ids = topk_ids[begin:end]
        curr_w = topk_weights[begin:end]
        # the workspace first: with blocks of 256 the alignment also leaves the large-tile
        # kernel's per-XCD ranges and cleared counters in it (one launch less)
        ws_bytes = L.moe_fused_experts_workspace_bytes(tokens_in_chunk, w1.size(2), N // 2, global_num_experts,
                                                       top_k_num, bm, act_code, weight_code)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        plan = None
        if global_num_experts == E:
            plan = _plan_in_workspace(workspace, tokens_in_chunk, w1.size(2), N // 2, E, top_k_num, bm,
                                      act_code, weight_code, curr_ids.numel())
        if _route is not None:
            # routing and alignment as one launch (fused_topk_experts): topk_weights / topk_ids
            # are this call's own buffers and are filled here, in front of their first use
            sorted_token_ids, expert_ids, num_tokens_post_padded = _route_align_block_size(
                _route[0], _route[1], curr_w, curr_ids, bm, global_num_experts, plan)
        else:
            sorted_token_ids, expert_ids, num_tokens_post_padded = _align_block_size(
                curr_ids, bm, global_num_experts, plan)
        args = launch_fused_experts(hidden_states[begin:end], out_hidden_states[begin:end], w1, w2,
                                    w1_bias, w2_bias, w1_scale, w2_scale, curr_w, sorted_token_ids,
                                    expert_ids, num_tokens_post_padded, bm, activation,
                                    apply_router_weight_on_input, weight_code=weight_code,
                                    workspace=workspace, passes=16 if plan is not None else 0,
                                    weight_layout=weight_layout)
        if _CHECK_HANDOFF and not torch.cuda.is_current_stream_capturing():  # the check waits for the stream
            fused_experts_status(args)
    return out_hidden_states

