"""ctypes binding of libmoe_gfx950.so (the C ABI declared in include/moe_gfx950.h).

There is no fallback: if the shared library is missing or does not export a
symbol, importing the ops fails with an error that says how to build it.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libmoe_gfx950.so")
CSRC_DIR = os.path.join(_PKG_DIR, "csrc")

# MoeDtype / MoeIdDtype / MoeActivation of include/moe_gfx950.h
DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
E4M3_CODE = 3
ID_DTYPE_CODE = {torch.int32: 0, torch.int64: 1, torch.int16: 2, torch.int8: 3, torch.uint8: 4}
ACTIVATION_CODE = {"silu": 0, "swigluoai": 1, "gelu": 2}
WEIGHT_LAYOUT_CODE = {"plain": 0, "tiled": 1}   # MoeWeightLayout

EXPORTS = (
    "moe_last_error", "moe_abi_version", "moe_topk_softmax", "moe_align_workspace_bytes",
    "moe_align_block_size", "moe_silu_and_mul", "moe_swigluoai_and_mul", "moe_sum",
    "moe_fused_experts_workspace_bytes", "moe_fused_experts", "moe_preferred_block_size",
    "moe_quant_rows_e4m3", "moe_gate_topk_softmax", "moe_add_rms_norm",
    "moe_align_can_plan", "moe_align_block_size_planned", "moe_fused_experts_plan_layout",
    "moe_fused_experts_status", "moe_fused_experts_set_wait_limit", "moe_align_block_size_static",
    "moe_tile_expert_weights", "moe_tile_expert_weights_supported",
    "moe_route_align_supported", "moe_route_align_block_size",
)


class MoeFusedExpertsArgs(ctypes.Structure):
    _fields_ = [
        ("x", ctypes.c_void_p), ("out", ctypes.c_void_p), ("w13", ctypes.c_void_p),
        ("w2", ctypes.c_void_p), ("w13_bias", ctypes.c_void_p), ("w2_bias", ctypes.c_void_p),
        ("w13_scale", ctypes.c_void_p), ("w2_scale", ctypes.c_void_p),
        ("topk_weights", ctypes.c_void_p), ("sorted_token_ids", ctypes.c_void_p),
        ("expert_ids", ctypes.c_void_p), ("num_tokens_post_pad", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_int64),
        ("w13_stride_e", ctypes.c_int64), ("w13_stride_n", ctypes.c_int64),
        ("w2_stride_e", ctypes.c_int64), ("w2_stride_n", ctypes.c_int64),
        ("T", ctypes.c_int32), ("H", ctypes.c_int32), ("I", ctypes.c_int32),
        ("E", ctypes.c_int32), ("K", ctypes.c_int32), ("block_size", ctypes.c_int32),
        ("sorted_cap", ctypes.c_int64), ("act_dtype", ctypes.c_int32),
        ("weight_dtype", ctypes.c_int32), ("activation", ctypes.c_int32),
        ("apply_router_weight_on_input", ctypes.c_int32),
        ("swiglu_alpha", ctypes.c_float), ("swiglu_limit", ctypes.c_float),
        ("passes", ctypes.c_int32), ("weight_layout", ctypes.c_int32), ("stream", ctypes.c_void_p),
    ]


_lib: Optional[ctypes.CDLL] = None


def build_library(verbose: bool = False) -> str:
    """Compile csrc/*.hip into libmoe_gfx950.so with hipcc (cross-compiles
    without a GPU)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(["make", "-C", CSRC_DIR, "-B", "-j8"], stdout=out, stderr=out)
    return LIB_PATH


def _declare(L: ctypes.CDLL) -> None:
    p, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
    L.moe_last_error.restype = ctypes.c_char_p
    L.moe_last_error.argtypes = []
    L.moe_abi_version.restype = i32
    L.moe_topk_softmax.restype = i32
    L.moe_topk_softmax.argtypes = [p, p, p, p, i32, i32, i32, i32, p]
    L.moe_gate_topk_softmax.restype = i32
    L.moe_gate_topk_softmax.argtypes = [p, p, i32, p, p, p, p, i32, i32, i32, i32, i32, p]
    L.moe_align_workspace_bytes.restype = i64
    L.moe_align_workspace_bytes.argtypes = [i64, i32]
    L.moe_align_block_size.restype = i32
    L.moe_align_block_size.argtypes = [p, i32, i64, i32, i32, p, i64, p, i64, p, p, i64, p]
    L.moe_align_block_size_static.restype = i32
    L.moe_align_block_size_static.argtypes = [p, i32, i64, i32, i32, p, i64, p, i64, p, p]
    L.moe_align_can_plan.restype = i32
    L.moe_align_can_plan.argtypes = [i64, i32]
    L.moe_align_block_size_planned.restype = i32
    L.moe_align_block_size_planned.argtypes = [p, i32, i64, i32, i32, p, i64, p, i64, p, p, i64, p, p, p, i32, i32]
    L.moe_fused_experts_plan_layout.restype = i32
    L.moe_fused_experts_plan_layout.argtypes = [i32] * 8 + [ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64),
                                                            ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]
    L.moe_silu_and_mul.restype = i32
    L.moe_silu_and_mul.argtypes = [p, p, i64, i32, i32, p]
    L.moe_swigluoai_and_mul.restype = i32
    L.moe_swigluoai_and_mul.argtypes = [p, p, i64, i32, i32, f32, f32, p]
    L.moe_sum.restype = i32
    L.moe_sum.argtypes = [p, p, i64, i32, i32, i32, p]
    L.moe_fused_experts_workspace_bytes.restype = i64
    L.moe_fused_experts_workspace_bytes.argtypes = [i32] * 8
    L.moe_fused_experts.restype = i32
    L.moe_fused_experts.argtypes = [ctypes.POINTER(MoeFusedExpertsArgs)]
    L.moe_fused_experts_status.restype = i32
    L.moe_fused_experts_status.argtypes = [ctypes.POINTER(MoeFusedExpertsArgs)]
    L.moe_fused_experts_set_wait_limit.restype = i32
    L.moe_fused_experts_set_wait_limit.argtypes = [i32]
    L.moe_preferred_block_size.restype = i32
    L.moe_preferred_block_size.argtypes = [i32] * 5
    L.moe_quant_rows_e4m3.restype = i32
    L.moe_quant_rows_e4m3.argtypes = [p, i32, i64, i32, p, p, p]
    L.moe_route_align_supported.restype = i32
    L.moe_route_align_supported.argtypes = [i32, i32, i32]
    L.moe_route_align_block_size.restype = i32
    L.moe_route_align_block_size.argtypes = [p, p, p, p, i32, i32, i32, i32, i32, p, i64, p, i64, p, p, p, p, i32, i32]
    L.moe_tile_expert_weights_supported.restype = i32
    L.moe_tile_expert_weights_supported.argtypes = [i32] * 4
    L.moe_tile_expert_weights.restype = i32
    L.moe_tile_expert_weights.argtypes = [p, p, i32, i32, i32, i32, i32, i32, p]
    L.moe_add_rms_norm.restype = i32
    L.moe_add_rms_norm.argtypes = [p, i64, p, i64, p, i64, p, i32, i64, i32, f32, p]


def lib() -> ctypes.CDLL:
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension has not been built. "
                f"Run `make -C {CSRC_DIR}` (or __graft_entry__.build()). There is no "
                "CPU or PyTorch fallback for these ops.")
        L = ctypes.CDLL(LIB_PATH)
        missing = [s for s in EXPORTS if not hasattr(L, s)]
        if missing:
            raise RuntimeError(f"{LIB_PATH} lacks symbols {missing}; rebuild it")
        _declare(L)
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(lib().moe_last_error().decode())


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu_tensor(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} is on {t.device}: these ops run only on an AMD GPU through "
            "libmoe_gfx950.so (there is no CPU path)")
