"""Fills ``FusedMoE`` layers from a Hugging Face safetensors checkpoint: the
expert part of the reference's ``nanovllm/utils/loader.py:37-93`` (name pattern
at :37-40, projection table at :42-50, per-tensor dispatch at :64-93).  Only
expert tensors are handled; every other name is handed back to the caller.
MX-FP4 block tensors (``*_blocks`` / ``*_scales``, :52-62,72-88) need the
amd-quark dequantiser, which is not part of this build, and are rejected."""
from __future__ import annotations

import glob
import os
import re
from typing import Callable, Dict, Iterable, Iterator, List, Optional, Tuple

import torch

from .layer import FusedMoE

MOE_EXPERT_PATTERN = re.compile(
    r"^model\.layers\.(\d+)\.mlp\.experts(?:\.(\d+))?\."
    r"(down_proj|up_proj|gate_proj|down_proj_bias|gate_up_proj_bias|gate_up_proj_blocks|down_proj_blocks)"
    r"(?:\.weight)?$")

# checkpoint projection -> (parameter of FusedMoE, shard id for weight_loader)
PROJ_TO_PARAM_SHARD: Dict[str, Tuple[str, str]] = {
    "down_proj": ("w2_weight", "w2"),
    "gate_proj": ("w13_weight", "w1"),
    "up_proj": ("w13_weight", "w3"),
    "gate_up_proj_bias": ("w13_bias", "w13"),
    "down_proj_bias": ("w2_bias", "w2"),
}


def load_expert_tensor(layers: Callable[[int], Optional[FusedMoE]], name: str,
                       tensor: torch.Tensor) -> bool:
    """Routes one checkpoint tensor.  Returns False when `name` is not an
    expert tensor (the caller loads it some other way)."""
    m = MOE_EXPERT_PATTERN.fullmatch(name)
    if m is None:
        return False
    layer_idx, expert, proj = int(m.group(1)), m.group(2), m.group(3)
    if proj not in PROJ_TO_PARAM_SHARD:
        raise NotImplementedError(f"{name}: MX-FP4 block tensors need a dequantiser this build lacks")
    layer = layers(layer_idx)
    assert layer is not None, f"FusedMoE layer not found for layer index {layer_idx}"
    param_name, shard_id = PROJ_TO_PARAM_SHARD[proj]
    if expert is None:
        # one tensor for all experts (gpt-oss style): dimension 0 is the expert
        shard_id = "all" if tensor.dim() == layer.get_parameter(param_name).dim() and \
            layer.tp_size == 1 else shard_id
    layer.weight_loader(layer.get_parameter(param_name), tensor, name, shard_id,
                        int(expert) if expert is not None else 0)
    return True


def iter_safetensors(path: str) -> Iterator[Tuple[str, torch.Tensor]]:
    from safetensors import safe_open
    for file in sorted(glob.glob(os.path.join(path, "*.safetensors"))):
        with safe_open(file, "pt", "cpu") as f:
            for name in f.keys():
                yield name, f.get_tensor(name)


def load_moe_experts(layers: Callable[[int], Optional[FusedMoE]],
                     tensors: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
    """Loads every expert tensor of `tensors` (name, tensor pairs, e.g.
    ``iter_safetensors(path)``); returns the names it did not consume."""
    rest = []
    for name, tensor in tensors:
        if not load_expert_tensor(layers, name, tensor):
            rest.append(name)
    return rest
