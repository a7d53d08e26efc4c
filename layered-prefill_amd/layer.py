"""``FusedMoE`` module with the interface of the reference's
``nanovllm/layers/fused_moe.py`` (types at :23-57, UnquantizedFusedMoEMethod at
:108-216, FusedMoE.__init__/select_experts/forward at :218-320,693-787, the
checkpoint loader at :330-658 and ``make_expert_params_mapping`` at :789-821),
on top of the HIP expert path.  TP=1 only at run time: the reference's optional
all-reduce (:746-748,782-785) belongs to its custom_all_reduce layer and is not
part of this build, so ``reduce_results=True`` with more than one rank raises.
The loader does slice for a tensor-parallel rank, as the reference's does.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Optional

import torch
import torch.distributed as dist

from . import ops
from .fused_moe import fused_experts, fused_gate_topk, fused_topk, fused_topk_experts


@dataclass
class FusedMoEParallelConfig:
    tp_size: int
    tp_rank: int

    @staticmethod
    def make() -> "FusedMoEParallelConfig":
        # nanovllm/layers/fused_moe.py:28-32 reads the default process group; a
        # process that never initialised one is a single rank.
        if dist.is_available() and dist.is_initialized():
            return FusedMoEParallelConfig(tp_size=dist.get_world_size(), tp_rank=dist.get_rank())
        return FusedMoEParallelConfig(tp_size=1, tp_rank=0)


@dataclass
class MoEConfig:
    num_experts: int
    experts_per_token: int
    hidden_dim: int
    num_local_experts: int
    moe_parallel_config: FusedMoEParallelConfig
    in_dtype: torch.dtype
    quant_dtype: Optional[torch.dtype] = None
    block_size: int = 128
    max_num_tokens: int = 256

    @property
    def tp_size(self) -> int:
        return self.moe_parallel_config.tp_size

    @property
    def tp_rank(self) -> int:
        return self.moe_parallel_config.tp_rank


class UnquantizedFusedMoEMethod:
    """nanovllm/layers/fused_moe.py:108-216."""

    def __init__(self, moe: MoEConfig):
        self.fused_experts = fused_experts
        self.topk_indices_dtype = None
        self.moe = moe

    def create_weights(self, layer: torch.nn.Module, num_experts: int, hidden_size: int,
                       intermediate_size_per_partition: int, params_dtype: torch.dtype,
                       has_bias: bool = False, **extra_weight_attrs) -> None:
        def _register(name: str, tensor: torch.Tensor) -> None:
            param = torch.nn.Parameter(tensor, requires_grad=False)
            layer.register_parameter(name, param)
            for key, value in extra_weight_attrs.items():
                setattr(param, key, value)

        # gate rows [0, I) then up rows [I, 2I) (nanovllm/layers/fused_moe.py:119-131,398-414)
        _register("w13_weight", torch.empty(num_experts, 2 * intermediate_size_per_partition,
                                            hidden_size, dtype=params_dtype))
        if has_bias:
            _register("w13_bias", torch.zeros(num_experts, 2 * intermediate_size_per_partition,
                                              dtype=params_dtype))
        _register("w2_weight", torch.empty(num_experts, hidden_size,
                                           intermediate_size_per_partition, dtype=params_dtype))
        if has_bias:
            _register("w2_bias", torch.zeros(num_experts, hidden_size, dtype=params_dtype))

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, router_logits: torch.Tensor,
              top_k: int, renormalize: bool, use_grouped_topk: bool = False,
              topk_group: Optional[int] = None, num_expert_group: Optional[int] = None,
              global_num_experts: int = -1, expert_map: Optional[torch.Tensor] = None,
              custom_routing_function: Optional[Callable] = None, scoring_func: str = "softmax",
              e_score_correction_bias: Optional[torch.Tensor] = None,
              apply_router_weight_on_input: bool = False, activation: str = "silu",
              expert_load_view: Optional[torch.Tensor] = None,
              logical_to_physical_map: Optional[torch.Tensor] = None,
              logical_replica_count: Optional[torch.Tensor] = None) -> torch.Tensor:
        layout = "tiled" if getattr(layer, "weights_tiled", False) else "plain"
        if (custom_routing_function is None and not use_grouped_topk and scoring_func == "softmax"
                and e_score_correction_bias is None and expert_map is None
                and self.topk_indices_dtype is None and self.fused_experts is fused_experts):
            # plain softmax routing: select_experts + fused_experts as one function, which
            # enqueues routing and alignment of a batch of up to 32 tokens as one launch
            return fused_topk_experts(
                x, router_logits, layer.w13_weight, layer.w2_weight, top_k, renormalize,
                w1_bias=layer.w13_bias if hasattr(layer, "w13_bias") else None,
                w2_bias=layer.w2_bias if hasattr(layer, "w2_bias") else None,
                inplace=True, activation=activation,
                apply_router_weight_on_input=apply_router_weight_on_input, weight_layout=layout)
        topk_weights, topk_ids = FusedMoE.select_experts(
            hidden_states=x, router_logits=router_logits, use_grouped_topk=use_grouped_topk,
            top_k=top_k, renormalize=renormalize, topk_group=topk_group,
            num_expert_group=num_expert_group, custom_routing_function=custom_routing_function,
            scoring_func=scoring_func, e_score_correction_bias=e_score_correction_bias,
            indices_type=self.topk_indices_dtype)
        return self.fused_experts(
            hidden_states=x, w1=layer.w13_weight, w2=layer.w2_weight,
            w1_bias=layer.w13_bias if hasattr(layer, "w13_bias") else None,
            w2_bias=layer.w2_bias if hasattr(layer, "w2_bias") else None,
            topk_weights=topk_weights, topk_ids=topk_ids, inplace=True, activation=activation,
            apply_router_weight_on_input=apply_router_weight_on_input,
            global_num_experts=global_num_experts, expert_map=expert_map, weight_layout=layout)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        """With ``FusedMoE(weight_layout="tiled")``: re-orders ``w13_weight`` and ``w2_weight`` once,
        after the checkpoint is in, into the unit order the DMA kernels fetch sequentially
        (``ops.tile_expert_weights``).  The parameters keep their shape and dtype but no longer
        hold weight [e, r, k] at [e, r, k]; ``layer.weights_tiled`` records it and ``apply`` hands
        it on.  The reference has no such step: its loader
        (nanovllm/layers/fused_moe.py:472-658) leaves the tensors row-major and only this layer
        reads them.  Shapes the tiling does not take (I not a multiple of 128, H not a multiple
        of 256, fp32) stay row-major."""
        from . import ops
        if getattr(layer, "weight_layout", "plain") != "tiled" or getattr(layer, "weights_tiled", False):
            return
        w13, w2 = layer.w13_weight.data, layer.w2_weight.data
        if not (w13.is_cuda and ops.tile_expert_weights_supported(w13, True)
                and ops.tile_expert_weights_supported(w2, False)):
            return
        interleaved = layer.activation == "swigluoai"
        layer.w13_weight.data = ops.tile_expert_weights(w13, True, interleaved)
        layer.w2_weight.data = ops.tile_expert_weights(w2, False)
        layer.weights_tiled = True


class Fp8E4M3FusedMoEMethod(UnquantizedFusedMoEMethod):
    """Per-output-channel e4m3 weights with dynamic per-token e4m3 activations.
    No counterpart in the reference (its ``fused_experts`` asserts the scale
    arguments are None, nanovllm/layers/for_moe/fused_moe.py:248-249); this is
    where the one-time weight quantisation lives.  Weights are created and
    loaded in ``params_dtype`` exactly like the unquantised method;
    ``process_weights_after_loading`` then replaces them by e4m3 codes and adds
    ``w13_weight_scale [E, 2I]`` / ``w2_weight_scale [E, H]`` (fp32)."""

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        from .fused_moe import quantize_expert_weights
        w13q, w13s, w2q, w2s = quantize_expert_weights(layer.w13_weight.data, layer.w2_weight.data)
        layer.w13_weight = torch.nn.Parameter(w13q, requires_grad=False)
        layer.w2_weight = torch.nn.Parameter(w2q, requires_grad=False)
        layer.register_parameter("w13_weight_scale", torch.nn.Parameter(w13s, requires_grad=False))
        layer.register_parameter("w2_weight_scale", torch.nn.Parameter(w2s, requires_grad=False))

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, router_logits: torch.Tensor,
              top_k: int, renormalize: bool, activation: str = "silu",
              apply_router_weight_on_input: bool = False, global_num_experts: int = -1,
              expert_map: Optional[torch.Tensor] = None,
              custom_routing_function: Optional[Callable] = None, **unused) -> torch.Tensor:
        if not hasattr(layer, "w13_weight_scale"):
            raise RuntimeError("Fp8E4M3FusedMoEMethod.apply before process_weights_after_loading")
        topk_weights, topk_ids = FusedMoE.select_experts(
            hidden_states=x, router_logits=router_logits, use_grouped_topk=False, top_k=top_k,
            renormalize=renormalize, custom_routing_function=custom_routing_function,
            indices_type=self.topk_indices_dtype)
        return self.fused_experts(
            hidden_states=x, w1=layer.w13_weight, w2=layer.w2_weight,
            w1_bias=layer.w13_bias if hasattr(layer, "w13_bias") else None,
            w2_bias=layer.w2_bias if hasattr(layer, "w2_bias") else None,
            topk_weights=topk_weights, topk_ids=topk_ids, inplace=True, activation=activation,
            apply_router_weight_on_input=apply_router_weight_on_input, per_channel_quant=True,
            global_num_experts=global_num_experts, expert_map=expert_map,
            w1_scale=layer.w13_weight_scale, w2_scale=layer.w2_weight_scale)


class FusedMoE(torch.nn.Module):
    """nanovllm/layers/fused_moe.py:218-320,330-658,693-821."""

    def __init__(self, num_experts: int, top_k: int, hidden_size: int, intermediate_size: int,
                 params_dtype: Optional[torch.dtype] = None, reduce_results: bool = False,
                 renormalize: bool = True, use_grouped_topk: bool = False,
                 num_expert_group: Optional[int] = None, topk_group: Optional[int] = None,
                 tp_size: Optional[int] = None, ep_size: Optional[int] = None,
                 dp_size: Optional[int] = None, prefix: str = "",
                 custom_routing_function: Optional[Callable] = None,
                 scoring_func: str = "softmax",
                 e_score_correction_bias: Optional[torch.Tensor] = None,
                 apply_router_weight_on_input: bool = False, activation: str = "silu",
                 num_redundant_experts: int = 0, has_bias: bool = False,
                 quantization: Optional[str] = None, weight_layout: str = "plain"):
        super().__init__()
        if params_dtype is None:
            params_dtype = torch.get_default_dtype()
        self.params_dtype = params_dtype
        self.moe_parallel_config = FusedMoEParallelConfig.make()
        self.global_num_experts = num_experts + num_redundant_experts
        self.layer_name = prefix
        self.expert_load_view = None
        self.logical_to_physical_map = None
        self.logical_replica_count = None
        self.local_num_experts, self.expert_map = self.global_num_experts, None
        self.top_k = top_k
        assert intermediate_size % self.tp_size == 0
        self.hidden_size = hidden_size
        self.intermediate_size_per_partition = intermediate_size // self.tp_size
        self.reduce_results = reduce_results
        self.renormalize = renormalize
        self.use_grouped_topk = use_grouped_topk
        if self.use_grouped_topk:
            assert num_expert_group is not None and topk_group is not None
        self.num_expert_group = num_expert_group
        self.topk_group = topk_group
        self.custom_routing_function = custom_routing_function
        self.scoring_func = scoring_func
        self.e_score_correction_bias = e_score_correction_bias
        self.apply_router_weight_on_input = apply_router_weight_on_input
        self.activation = activation
        # `weight_layout` has no counterpart in the reference constructor: "tiled" makes
        # process_weights_after_loading re-order the expert weights for the DMA kernels
        if weight_layout not in ("plain", "tiled"):
            raise ValueError(f"unsupported weight_layout {weight_layout!r}")
        self.weight_layout = weight_layout
        self.weights_tiled = False
        if self.scoring_func != "softmax" and not self.use_grouped_topk:
            raise ValueError("Only softmax scoring function is supported for non-grouped topk.")
        self.moe_config = MoEConfig(
            num_experts=self.global_num_experts, experts_per_token=top_k, hidden_dim=hidden_size,
            num_local_experts=self.local_num_experts,
            moe_parallel_config=self.moe_parallel_config, in_dtype=params_dtype,
            quant_dtype=params_dtype, max_num_tokens=256)
        # `quantization` has no counterpart in the reference constructor (it only
        # builds the unquantised method, :300-304); "fp8_e4m3" selects the e4m3 path
        if quantization is None:
            self.quant_method = UnquantizedFusedMoEMethod(self.moe_config)
        elif quantization == "fp8_e4m3":
            self.quant_method = Fp8E4M3FusedMoEMethod(self.moe_config)
        else:
            raise ValueError(f"unsupported quantization {quantization!r}")
        self.quant_method.create_weights(
            layer=self, num_experts=self.local_num_experts, hidden_size=hidden_size,
            intermediate_size_per_partition=self.intermediate_size_per_partition,
            params_dtype=params_dtype, has_bias=has_bias, weight_loader=self.weight_loader)

    # ------------------------------------------------------------------ checkpoint loading
    _SHARDED_DIM = {"w1": 0, "w2": 1, "w3": 0, "w13": 1}

    def _tp_slice(self, tensor: torch.Tensor, dim: int, size: int) -> torch.Tensor:
        """This rank's `size` entries of `tensor` along `dim`."""
        return tensor.narrow(dim, size * self.tp_rank, size)

    def _load_w13(self, expert_data: torch.Tensor, shard_dim: int, shard_id: str,
                  loaded_weight: torch.Tensor) -> None:
        # gate_proj fills the first half of w13 along shard_dim, up_proj the second
        # (nanovllm/layers/fused_moe.py:398-414); column-parallel over the rank
        half = expert_data.shape[shard_dim] // 2
        src = self._tp_slice(loaded_weight, shard_dim, half)
        expert_data.narrow(shard_dim, 0 if shard_id == "w1" else half, half).copy_(src)

    def _load_w2(self, expert_data: torch.Tensor, shard_dim: int,
                 loaded_weight: torch.Tensor) -> None:
        # down_proj is row-parallel: the rank keeps its slice of the input dimension
        # (nanovllm/layers/fused_moe.py:416-432)
        expert_data.copy_(self._tp_slice(loaded_weight, shard_dim, expert_data.shape[shard_dim]))

    def _load_matrix(self, shard_id: str, shard_dim: int, expert_data: torch.Tensor,
                     loaded_weight: torch.Tensor) -> None:
        if expert_data.ndim != loaded_weight.ndim:
            loaded_weight = loaded_weight.reshape(*loaded_weight.shape[:-2], -1)
        if shard_id == "w2":
            self._load_w2(expert_data, shard_dim, loaded_weight)
        elif shard_id in ("w1", "w3"):
            self._load_w13(expert_data, shard_dim, shard_id, loaded_weight)
        else:  # "w13": gate and up already merged in the checkpoint
            size = expert_data.shape[1]
            expert_data.narrow(1, 0, size).copy_(loaded_weight.narrow(1, size * self.tp_rank, size))

    def weight_loader(self, param: torch.nn.Parameter, loaded_weight: torch.Tensor,
                      weight_name: str, shard_id: str, expert_id: int,
                      return_success: bool = False) -> Optional[bool]:
        """Copies one checkpoint tensor into its place in ``w13_weight`` /
        ``w2_weight`` (or a bias / per-channel scale), same contract as
        nanovllm/layers/fused_moe.py:472-658: ``shard_id`` is ``w1`` (gate_proj),
        ``w3`` (up_proj), ``w2`` (down_proj), ``w13`` (merged gate_up) or ``all``
        (all experts in one tensor); tensors are sliced for this TP rank.
        Checkpoint formats the reference routes to other quantisation methods
        (GGUF, g_idx, ModelOpt, group/block/tensor scales, input scales) are
        rejected: no such method exists on this path."""
        ok = True if return_success else None
        if shard_id == "all":
            if "bias" in weight_name:
                param.data.copy_(loaded_weight)
            else:
                param.data.copy_(loaded_weight.reshape(*param.data.shape[:-1], -1))
            return ok
        if self.expert_map is not None:
            expert_id = int(self.expert_map[expert_id])
            if expert_id == -1:
                return False if return_success else None
        if shard_id not in self._SHARDED_DIM:
            raise ValueError(f"shard_id must be ['w1','w2','w3', 'all'] but got {shard_id}.")
        for marker in ("input_scale", "g_idx", "weight_shape", "zero", "offset"):
            if marker in weight_name:
                raise ValueError(f"{weight_name}: '{marker}' tensors belong to quantisation "
                                 "methods this layer does not have")
        shard_dim = self._SHARDED_DIM[shard_id]
        if getattr(param, "is_transposed", False):
            shard_dim = 1 - shard_dim
        full_load = loaded_weight.dim() == 3 or "bias" in weight_name
        if full_load:
            shard_dim += 1
        expert_data = param.data if full_load else param.data[expert_id]
        if "scale" in weight_name:
            # per-output-channel weight scales of the e4m3 method: a vector per expert
            if shard_id == "w2":
                expert_data.copy_(loaded_weight)
            else:
                self._load_w13(expert_data, shard_dim, shard_id, loaded_weight)
            return ok
        if "weight" in weight_name:
            self._load_matrix(shard_id, shard_dim, expert_data, loaded_weight)
            return ok
        if "bias" in weight_name:
            if shard_id == "w2":
                # the down bias is added once: only rank 0 keeps it
                if self.tp_rank == 0:
                    expert_data.copy_(loaded_weight)
                else:
                    expert_data.zero_()
            else:
                n = loaded_weight.size(-1) // self.tp_size
                expert_data.copy_(loaded_weight.narrow(-1, self.tp_rank * n, n))
            return ok
        raise ValueError(f"Unrecognized weight_name {weight_name}.")

    @classmethod
    def make_expert_params_mapping(cls, ckpt_gate_proj_name: str, ckpt_down_proj_name: str,
                                   ckpt_up_proj_name: str, num_experts: int,
                                   num_redundant_experts: int = 0) -> list:
        """``(param_name, weight_name, expert_id, shard_id)`` for every physical
        expert and projection (nanovllm/layers/fused_moe.py:789-821); redundant
        experts replay the logical ones round-robin."""
        logical = list(range(num_experts)) + [i % num_experts for i in range(num_redundant_experts)]
        mapping = []
        for expert_id, logical_id in enumerate(logical):
            for shard_id, name in (("w1", ckpt_gate_proj_name), ("w2", ckpt_down_proj_name),
                                   ("w3", ckpt_up_proj_name)):
                param = "experts.w13_" if name in (ckpt_gate_proj_name, ckpt_up_proj_name) else "experts.w2_"
                mapping.append((param, f"experts.{logical_id}.{name}.", expert_id, shard_id))
        return mapping

    def process_weights_after_loading(self) -> None:
        hook = getattr(self.quant_method, "process_weights_after_loading", None)
        if hook is not None:
            hook(self)

    @property
    def tp_size(self) -> int:
        return self.moe_parallel_config.tp_size

    @property
    def tp_rank(self) -> int:
        return self.moe_parallel_config.tp_rank

    @staticmethod
    def select_experts(hidden_states: torch.Tensor, router_logits: torch.Tensor, top_k: int,
                       use_grouped_topk: bool, renormalize: bool,
                       topk_group: Optional[int] = None, num_expert_group: Optional[int] = None,
                       custom_routing_function: Optional[Callable] = None,
                       scoring_func: str = "softmax",
                       e_score_correction_bias: Optional[torch.Tensor] = None,
                       indices_type: Optional[torch.dtype] = None,
                       expert_map: Optional[torch.Tensor] = None,
                       expert_load_view: Optional[torch.Tensor] = None,
                       logical_to_physical_map: Optional[torch.Tensor] = None,
                       logical_replica_count: Optional[torch.Tensor] = None):
        """nanovllm/layers/fused_moe.py:693-741."""
        if custom_routing_function is None:
            topk_weights, topk_ids, _ = fused_topk(hidden_states=hidden_states,
                                                   gating_output=router_logits, topk=top_k,
                                                   renormalize=renormalize)
        else:
            topk_weights, topk_ids = custom_routing_function(
                hidden_states=hidden_states, gating_output=router_logits, topk=top_k,
                renormalize=renormalize)
            if indices_type is not None:
                topk_ids = topk_ids.to(dtype=indices_type)
        return topk_weights, topk_ids

    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
        final_hidden_states = self.quant_method.apply(
            layer=self, x=hidden_states, router_logits=router_logits, top_k=self.top_k,
            renormalize=self.renormalize, use_grouped_topk=self.use_grouped_topk,
            global_num_experts=self.global_num_experts, expert_map=self.expert_map,
            topk_group=self.topk_group, num_expert_group=self.num_expert_group,
            custom_routing_function=self.custom_routing_function, scoring_func=self.scoring_func,
            e_score_correction_bias=self.e_score_correction_bias, activation=self.activation,
            apply_router_weight_on_input=self.apply_router_weight_on_input)
        if self.reduce_results and self.tp_size > 1:
            raise NotImplementedError(
                "tensor-parallel all-reduce of the expert output is outside this build (TP=1)")
        return final_hidden_states

    def extra_repr(self) -> str:
        return (f"global_num_experts={self.global_num_experts}, top_k={self.top_k}, "
                f"intermediate_size_per_partition={self.intermediate_size_per_partition}, "
                f"tp_size={self.tp_size}, renormalize={self.renormalize}, "
                f"scoring_func='{self.scoring_func}', activation='{self.activation}'")


class SparseMoeBlock(torch.nn.Module):
    """Router gate + experts, the shape of the reference's
    ``Qwen3MoeSparseMoeBlock`` (nanovllm/models/qwen3_moe.py:70-118): a bias-free
    gate ``[num_experts, hidden_size]`` (its ``ReplicatedLinear``) and a
    ``FusedMoE``.  ``forward(hidden_states)`` routes with the fused gate + top-k
    kernel when the shape allows and hands the experts the routing through
    ``custom_routing_function``-free plumbing: the result equals
    ``experts(x, gate(x))``.  TP=1 (the reference's all-reduce at :113-116 is
    outside this build)."""

    def __init__(self, num_experts: int, top_k: int, hidden_size: int, intermediate_size: int,
                 params_dtype: Optional[torch.dtype] = None, renormalize: bool = True,
                 activation: str = "silu", has_bias: bool = False,
                 quantization: Optional[str] = None):
        super().__init__()
        self.experts = FusedMoE(num_experts=num_experts, top_k=top_k, hidden_size=hidden_size,
                                intermediate_size=intermediate_size, params_dtype=params_dtype,
                                reduce_results=False, renormalize=renormalize,
                                activation=activation, has_bias=has_bias, quantization=quantization)
        self.gate_weight = torch.nn.Parameter(
            torch.empty(num_experts, hidden_size, dtype=self.experts.params_dtype), requires_grad=False)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        orig_shape = hidden_states.shape
        x = hidden_states.view(-1, orig_shape[-1])
        ex = self.experts
        topk_weights, topk_ids, _ = fused_gate_topk(x, self.gate_weight, ex.top_k, ex.renormalize)
        out = ex.quant_method.apply(
            layer=ex, x=x, router_logits=None, top_k=ex.top_k, renormalize=ex.renormalize,
            activation=ex.activation, apply_router_weight_on_input=ex.apply_router_weight_on_input,
            global_num_experts=ex.global_num_experts, expert_map=ex.expert_map,
            custom_routing_function=lambda **_: (topk_weights, topk_ids))
        return out.view(orig_shape)


class GptOssMLP(torch.nn.Module):
    """The gpt-oss form of the block, the shape of the reference's ``GptOssMLP``
    (nanovllm/models/gpt_oss.py:120-158): a router linear *with* bias and experts
    with ``w13_bias`` / ``w2_bias`` and the interleaved, clamped ``swigluoai``
    activation.  ``forward(x)`` = ``experts(x, router(x))``.  The router is a plain
    library GEMM (its bias keeps it off the fused gate kernel).  TP=1."""

    def __init__(self, num_local_experts: int, num_experts_per_tok: int, hidden_size: int,
                 intermediate_size: int, params_dtype: Optional[torch.dtype] = torch.bfloat16):
        super().__init__()
        self.num_experts = num_local_experts
        self.top_k = num_experts_per_tok
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.router = torch.nn.Linear(hidden_size, num_local_experts, dtype=params_dtype)
        self.experts = FusedMoE(num_experts=num_local_experts, top_k=num_experts_per_tok,
                                hidden_size=hidden_size, intermediate_size=intermediate_size,
                                params_dtype=params_dtype, reduce_results=False, renormalize=True,
                                has_bias=True, activation="swigluoai")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        g = self.router(x)
        return self.experts(hidden_states=x, router_logits=g)


class RMSNorm(torch.nn.Module):
    """The norm in front of the MoE block, same interface as the reference's
    ``RMSNorm`` (nanovllm/layers/layernorm.py:7-34): ``forward(x)`` returns the
    normalised tensor, ``forward(x, residual)`` adds ``x`` into ``residual`` in
    place first and returns ``(out, residual)``."""

    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.ones(hidden_size))

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None):
        if out is None:
            out = torch.empty_like(x)
        if residual is None:
            ops.rms_norm(out, x, self.weight.data, self.eps)
            return out
        ops.add_rms_norm(out, residual, x, self.weight.data, self.eps)
        return out, residual
