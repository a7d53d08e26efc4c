"""TEST INFRASTRUCTURE ONLY: CPU oracle for the fused-MoE expert path.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped package never does.

Two layers:

* bit-level functions (router softmax + top-k, expert-sorted alignment, gated
  activations) are the scalar C restatement in ``oracle/moe_oracle.c`` loaded
  through ctypes; each C function cites the reference lines it follows;
* the expert MLP itself is floating-point GEMM work and is restated here as a
  dense per-expert loop in fp32 torch (``fused_experts_ref``), following
  ``nanovllm/layers/for_moe/fused_moe.py:461-633`` (flow),
  ``:84-223`` (what one grouped-GEMM block computes),
  ``csrc/activation_kernels.cu:8-64`` (activations) and
  ``nanovllm/layers/for_moe/moe_easy_kernel.py:26-31`` (top-k combine).
  The reference does this arithmetic in Triton ``tl.dot`` (third-party, not in
  the reference tree, pinned only as ``triton>=3.0.0``) and ships no test or
  golden vector for it, so ``fused_experts_ref`` is pinned by the textbook
  special cases exercised in ``tests/test_oracle.py``: K=1 gated MLP, E=1 dense
  MLP, linearity in the routed weights, permutation invariance; every branch
  (both biases, gelu, swigluoai, routed weight on the input side, the top-k sum)
  against torch's float64 ``linear`` / ``silu`` / ``gelu`` per expert; both
  mirrored rounding modes step by step on a hand-sized case.  The *bits* of the
  reference's result (Triton's accumulation order) stay "parity unpinned".
* ``fused_experts_fp8_ref`` has no counterpart in the reference (it asserts the
  scales None); it is pinned as a definition: step by step against torch's own
  ``float8_e4m3fn`` cast and ``F.linear`` with non-uniform row and channel
  scales, and against ``fused_experts_ref`` on losslessly quantisable tensors up
  to the provable bound of the one re-quantisation.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmoe_oracle.so")
_lib = None

_ID_DTYPES = {torch.int32: 0, torch.int64: 1, torch.int16: 2, torch.int8: 3, torch.uint8: 4}


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmoe_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        c_p, c_i, c_l, c_f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
        L.oracle_expf.restype = c_f
        L.oracle_expf.argtypes = [c_f]
        L.oracle_expf_array.argtypes = [c_p, c_p, c_l]
        L.oracle_topk_softmax.restype = c_i
        L.oracle_topk_softmax.argtypes = [c_p, c_p, c_p, c_p, c_p, c_i, c_i, c_i, c_i]
        L.oracle_moe_align_block_size.restype = c_i
        L.oracle_moe_align_block_size.argtypes = [c_p, c_i, c_l, c_i, c_i, c_p, c_l, c_p, c_l, c_p]
        for name in ("oracle_silu_and_mul_f32", "oracle_silu_and_mul_bf16"):
            getattr(L, name).argtypes = [c_p, c_p, c_l, c_i]
        for name in ("oracle_swigluoai_and_mul_f32", "oracle_swigluoai_and_mul_bf16"):
            getattr(L, name).argtypes = [c_p, c_p, c_l, c_i, c_f, c_f]
        _lib = L
    return _lib


def _cpu(t: torch.Tensor) -> torch.Tensor:
    return t.detach().cpu().contiguous()


def expf(x: torch.Tensor) -> torch.Tensor:
    x = _cpu(x).float()
    y = torch.empty_like(x)
    lib().oracle_expf_array(x.data_ptr(), y.data_ptr(), x.numel())
    return y


def topk_softmax(gating_output: torch.Tensor, topk: int, renormalize: bool = False,
                 return_probs: bool = False):
    """csrc/moe_topk_softmax_kernels.cu:476-503 (+ renormalise of
    nanovllm/layers/for_moe/fused_moe.py:417-418 when asked).
    Returns (topk_weights f32[T,K], topk_ids i32[T,K], token_expert_indices i32[T,K])."""
    g = _cpu(gating_output).float()
    T, E = g.shape
    w = torch.empty(T, topk, dtype=torch.float32)
    ids = torch.empty(T, topk, dtype=torch.int32)
    tei = torch.empty(T, topk, dtype=torch.int32)
    probs = torch.empty(T, E, dtype=torch.float32) if return_probs else None
    rc = lib().oracle_topk_softmax(g.data_ptr(), w.data_ptr(), ids.data_ptr(), tei.data_ptr(),
                                   probs.data_ptr() if return_probs else None,
                                   T, E, topk, int(renormalize))
    if rc != 0:
        raise ValueError(f"oracle_topk_softmax rejected T={T} E={E} K={topk}")
    if return_probs:
        return w, ids, tei, probs
    return w, ids, tei


def fused_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int,
               renormalize: bool):
    """nanovllm/layers/for_moe/fused_moe.py:393-419."""
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    return topk_softmax(gating_output, topk, renormalize)


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int
                         ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """nanovllm/layers/for_moe/fused_moe.py:17-70 with the native op of
    csrc/moe_align_block_size_kernels.cu:239-291 (stable order)."""
    ids = _cpu(topk_ids)
    if ids.dtype not in _ID_DTYPES:
        raise TypeError(f"unsupported id dtype {ids.dtype}")
    numel = ids.numel()
    P = numel + num_experts * (block_size - 1)
    B = (P + block_size - 1) // block_size
    sorted_ids = torch.empty(P, dtype=torch.int32)
    expert_ids = torch.empty(B, dtype=torch.int32)
    npp = torch.empty(1, dtype=torch.int32)
    rc = lib().oracle_moe_align_block_size(ids.data_ptr(), _ID_DTYPES[ids.dtype], numel,
                                           num_experts, block_size, sorted_ids.data_ptr(), P,
                                           expert_ids.data_ptr(), B, npp.data_ptr())
    if rc != 0:
        raise ValueError(f"oracle_moe_align_block_size failed rc={rc}")
    return sorted_ids, expert_ids, npp


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """csrc/activation_kernels.cu:14-25: [rows, 2d] -> [rows, d]."""
    x = _cpu(x)
    rows, two_d = x.shape
    d = two_d // 2
    out = torch.empty(rows, d, dtype=x.dtype)
    if x.dtype == torch.float32:
        lib().oracle_silu_and_mul_f32(out.data_ptr(), x.data_ptr(), rows, d)
    elif x.dtype == torch.bfloat16:
        lib().oracle_silu_and_mul_bf16(out.data_ptr(), x.data_ptr(), rows, d)
    elif x.dtype == torch.float16:
        xf = x.float()
        s = torch.empty(rows, d, dtype=torch.float32)
        # T(silu(x)) * y with T = half: silu in fp32, cast, product rounded to half
        gate_and_ones = torch.cat([xf[:, :d], torch.ones(rows, d)], 1).contiguous()
        lib().oracle_silu_and_mul_f32(s.data_ptr(), gate_and_ones.data_ptr(), rows, d)
        out = (s.half().float() * xf[:, d:]).half()
    else:
        raise TypeError(x.dtype)
    return out


def swigluoai_and_mul(x: torch.Tensor, alpha: float = 1.702, limit: float = 7.0) -> torch.Tensor:
    """csrc/activation_kernels.cu:27-64: interleaved gate/up, [rows, 2d] -> [rows, d]."""
    x = _cpu(x)
    rows, two_d = x.shape
    d = two_d // 2
    out = torch.empty(rows, d, dtype=x.dtype)
    if x.dtype == torch.float32:
        lib().oracle_swigluoai_and_mul_f32(out.data_ptr(), x.data_ptr(), rows, d, alpha, limit)
    elif x.dtype == torch.bfloat16:
        lib().oracle_swigluoai_and_mul_bf16(out.data_ptr(), x.data_ptr(), rows, d, alpha, limit)
    elif x.dtype == torch.float16:
        o = torch.empty(rows, d, dtype=torch.float32)
        xf = x.float().contiguous()
        lib().oracle_swigluoai_and_mul_f32(o.data_ptr(), xf.data_ptr(), rows, d, alpha, limit)
        out = o.half()
    else:
        raise TypeError(x.dtype)
    return out


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """nanovllm/layers/for_moe/moe_easy_kernel.py:89-98 (erf GELU of the first
    half times the second half, in the tensor's dtype)."""
    d = x.shape[-1] // 2
    return torch.nn.functional.gelu(x[..., :d]) * x[..., d:]


# --------------------------------------------------------------------------
# fp8 e4m3fn (OCP) helpers, explicit so the rounding is not a library's choice
# --------------------------------------------------------------------------
E4M3_MAX = 448.0
E4M3_MIN_SCALE = 2.0 ** -100  # below it 1 / s would overflow for tiny non-zero rows


def _e4m3_table() -> np.ndarray:
    vals = np.zeros(256, dtype=np.float64)
    for b in range(256):
        s = -1.0 if b & 0x80 else 1.0
        e = (b >> 3) & 0xF
        m = b & 7
        if e == 0xF and m == 7:
            vals[b] = np.nan
        elif e == 0:
            vals[b] = s * (m / 8.0) * 2.0 ** -6
        else:
            vals[b] = s * (1 + m / 8.0) * 2.0 ** (e - 7)
    return vals


_E4M3 = _e4m3_table()
_E4M3_POS = _E4M3[:127].copy()  # 0 .. 448, ascending


def quant_e4m3(x: torch.Tensor) -> torch.Tensor:
    """fp32 -> e4m3fn codes (uint8): saturate to +-448, round to nearest even."""
    a = _cpu(x).float().numpy().astype(np.float64)
    sign = np.signbit(a)
    mag = np.minimum(np.abs(a), E4M3_MAX)
    hi = np.searchsorted(_E4M3_POS, mag, side="left").clip(0, 126)
    lo = np.maximum(hi - 1, 0)
    dlo = mag - _E4M3_POS[lo]
    dhi = _E4M3_POS[hi] - mag
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code = np.where(sign, code | 0x80, code).astype(np.uint8)
    return torch.from_numpy(code)


def dequant_e4m3(code: torch.Tensor) -> torch.Tensor:
    return torch.from_numpy(_E4M3[_cpu(code).numpy()].astype(np.float32))


def quant_weight_per_channel(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """[E, N, K] -> (codes uint8 [E,N,K], scales f32 [E,N]) with
    s[e,n] = max(amax_k |w[e,n,k]| / 448, 2^-100) (1.0 for an all-zero channel) and codes
    e4m3(w * (1 / s)), every operation a rounded fp32 one (the reciprocal form
    of dynamic fp8 quantisers: one division per row, one product per element)."""
    wf = _cpu(w).float()
    amax = wf.abs().amax(dim=-1)
    s = torch.where(amax > 0, torch.clamp(amax / E4M3_MAX, min=E4M3_MIN_SCALE), torch.ones_like(amax))
    q = quant_e4m3(wf * (1.0 / s)[..., None])
    return q, s


def quant_act_per_token(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """[R, K] -> (codes uint8, scales f32 [R]) with s[r] = amax|x[r]| / 448 and
    codes e4m3(x * (1 / s)), as ``quant_weight_per_channel``."""
    xf = _cpu(x).float()
    amax = xf.abs().amax(dim=-1)
    s = torch.where(amax > 0, torch.clamp(amax / E4M3_MAX, min=E4M3_MIN_SCALE), torch.ones_like(amax))
    q = quant_e4m3(xf * (1.0 / s)[:, None])
    return q, s


# --------------------------------------------------------------------------
# Expert MLP (floating point): dense per-expert restatement
# --------------------------------------------------------------------------
def _round(t: torch.Tensor, dtype: Optional[torch.dtype]) -> torch.Tensor:
    return t if dtype is None or dtype == torch.float32 else t.to(dtype).float()


def fused_experts_ref(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                      topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                      activation: str = "silu", apply_router_weight_on_input: bool = False,
                      w1_bias: Optional[torch.Tensor] = None,
                      w2_bias: Optional[torch.Tensor] = None,
                      mirror_rounding=False,
                      out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """out[t] = sum_k w[t,k] * W2[e] @ act(W13[e] @ x_t), e = ids[t,k].

    ``mirror_rounding=False``: pure fp32 (the authority the tolerances are
    stated against).  ``mirror_rounding=True``: round to the activation dtype at
    the points where the reference stores an intermediate (after GEMM1, after
    silu, after the gate*up product, after the routed-weight multiply, after
    the top-k sum; nanovllm/layers/for_moe/fused_moe.py:216,522-531,
    csrc/activation_kernels.cu:11,23), fp32 accumulation in between.
    ``mirror_rounding="fused"``: as ``True``, except that the SiLU-gated
    intermediate is rounded once, where a kernel that applies the activation to
    its fp32 accumulators stores it (no rounding after GEMM1 or after silu).
    """
    x = _cpu(hidden_states)
    dt = x.dtype if mirror_rounding else None
    fused_act = mirror_rounding == "fused" and activation == "silu"
    T, H = x.shape
    E, N, _ = w1.shape
    K = topk_ids.shape[1]
    xf = x.float()
    ids = _cpu(topk_ids).long()
    tw = _cpu(topk_weights).float()
    out_k = torch.zeros(T, K, w2.shape[1], dtype=torch.float32)
    for e in range(E):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        a = xf[tok]
        c1 = a @ _cpu(w1[e]).float().t()                      # fused_moe.py:191-205
        if w1_bias is not None:
            c1 = c1 + _cpu(w1_bias[e]).float()                # :207-208
        if apply_router_weight_on_input:
            c1 = c1 * tw[tok, slot, None]                     # :210-214 via :589
        c1 = _round(c1, None if fused_act else dt)            # :216
        if activation == "silu":
            if dt is None or fused_act:
                d = N // 2
                g, u = c1[:, :d], c1[:, d:]
                c2 = _round(g / (1 + torch.exp(-g)) * u, dt)
            else:
                c2 = silu_and_mul(c1.to(dt)).float()
        elif activation == "swigluoai":
            c2 = swigluoai_and_mul(c1.to(x.dtype) if dt is not None else c1).float()
        elif activation == "gelu":
            c2 = _round(gelu_and_mul(c1 if dt is None else c1.to(dt)).float(), dt)
        else:
            raise ValueError(f"Unsupported FusedMoe activation: {activation}")
        c3 = c2 @ _cpu(w2[e]).float().t()
        if w2_bias is not None:
            c3 = c3 + _cpu(w2_bias[e]).float()
        if not apply_router_weight_on_input:
            c3 = c3 * tw[tok, slot, None]                     # :210-214 via :621
        out_k[tok, slot] = _round(c3, dt)
    out = _round(out_k.sum(dim=1), dt)                         # moe_easy_kernel.py:26-31
    if out_dtype is not None:
        out = out.to(out_dtype)
    return out


def fused_experts_fp8_ref(hidden_states: torch.Tensor, w1_q: torch.Tensor, w1_scale: torch.Tensor,
                          w2_q: torch.Tensor, w2_scale: torch.Tensor,
                          topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                          mirror_rounding=False) -> torch.Tensor:
    """fp32 reference of the fp8 variant (not implemented by the reference:
    nanovllm/layers/for_moe/fused_moe.py:248-249,571,607 assert the scales are
    None): e4m3 per-output-channel weights, dynamic per-token e4m3 activations
    in front of both GEMMs, everything dequantised and multiplied in fp32.

    ``mirror_rounding=True`` additionally rounds to the activation dtype where
    the bf16 path stores an intermediate (GEMM1 result, silu, silu*up, weighted
    GEMM2 result, top-k sum), i.e. the second quantisation sees the stored
    16-bit intermediate rather than its fp32 value.  ``mirror_rounding="fused"``
    rounds that intermediate once (no rounding after GEMM1 or after silu)."""
    x16 = _cpu(hidden_states)
    dt = x16.dtype if mirror_rounding else None
    fused_act = mirror_rounding == "fused"
    x = x16.float()
    T, H = x.shape
    E, N, _ = w1_q.shape
    K = topk_ids.shape[1]
    ids = _cpu(topk_ids).long()
    tw = _cpu(topk_weights).float()
    xq, xs = quant_act_per_token(x)
    xd = dequant_e4m3(xq) * xs[:, None]
    out_k = torch.zeros(T, K, w2_q.shape[1], dtype=torch.float32)
    w1_q, w2_q = _cpu(w1_q).view(torch.uint8), _cpu(w2_q).view(torch.uint8)
    for e in range(E):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        W1 = dequant_e4m3(w1_q[e]) * _cpu(w1_scale[e]).float()[:, None]
        W2 = dequant_e4m3(w2_q[e]) * _cpu(w2_scale[e]).float()[:, None]
        c1 = xd[tok] @ W1.t()
        if dt is None or fused_act:
            d = N // 2
            g, u = c1[:, :d], c1[:, d:]
            c2 = _round(g / (1 + torch.exp(-g)) * u, dt)
        else:
            c2 = silu_and_mul(c1.to(dt)).float()
        cq, cs = quant_act_per_token(c2)
        c2d = dequant_e4m3(cq) * cs[:, None]
        out_k[tok, slot] = _round((c2d @ W2.t()) * tw[tok, slot, None], dt)
    return _round(out_k.sum(dim=1), dt)


def gate_logits(hidden_states: torch.Tensor, gate_weight: torch.Tensor) -> torch.Tensor:
    """Router logits as the reference's gate produces them: a bias-free linear in
    the activation dtype (nanovllm/models/qwen3_moe.py:93-104,113;
    nanovllm/layers/linear.py:53-60), i.e. the fp32 product rounded once to that
    dtype; returned upcast to fp32 as ``fused_topk`` feeds them to the softmax
    (nanovllm/layers/for_moe/fused_moe.py:409-415).  Pinned by the closed form
    against ``torch.nn.functional.linear`` in float64 (tests/test_oracle.py)."""
    acc = hidden_states.float() @ gate_weight.float().t()
    return acc.to(hidden_states.dtype).float()


def gate_topk_softmax(hidden_states: torch.Tensor, gate_weight: torch.Tensor, topk: int,
                      renormalize: bool = False):
    """``gate_logits`` followed by ``topk_softmax``."""
    return topk_softmax(gate_logits(hidden_states, gate_weight), topk, renormalize=renormalize)


def add_rms_norm(x: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor,
                 eps: float):
    """The norm in front of the MoE block, csrc/layernorm_kernels.cu:77-108
    (``add_rms_norm_kernel``) and :10-35 (``rms_norm_kernel``) of the reference:
    s = float(x) + float(residual); residual' = T(s); the variance is the mean of
    s*s over the row (s before rounding, :91-94); out = T(T(float(residual') * r) *
    weight) with r = rsqrt(variance + eps) (:97-107).  The mean is taken in float64
    here and r rounded to fp32 once, so results can differ from an fp32 reduction
    in the last place of r.  Returns ``(out, residual')`` (``residual'`` is None
    without a residual).  Pinned by known answers in tests/test_oracle.py."""
    dt = x.dtype
    s32 = x.float() if residual is None else x.float() + residual.float()
    new_res = None if residual is None else s32.to(dt)
    var = (s32.double() * s32.double()).mean(dim=-1, keepdim=True)
    r = (1.0 / torch.sqrt(var + float(eps))).float()
    base = s32 if residual is None else new_res.float()
    normed = (base * r).to(dt)
    out = (normed.float() * weight.float()).to(dt)
    return out, new_res
