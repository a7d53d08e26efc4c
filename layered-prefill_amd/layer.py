"""``FusedMoE`` module with the interface of the reference's
``nanovllm/layers/fused_moe.py`` (types at :23-57, UnquantizedFusedMoEMethod at
:108-216, FusedMoE.__init__/select_experts/forward at :218-320,693-787), on top
of the HIP expert path.  TP=1 only: the reference's optional all-reduce
(:746-748,782-785) belongs to its custom_all_reduce layer and is not part of
this build, so ``reduce_results=True`` with more than one rank raises.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Optional

import torch
import torch.distributed as dist

from .fused_moe import fused_experts, fused_topk


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
            global_num_experts=global_num_experts, expert_map=expert_map)


class FusedMoE(torch.nn.Module):
    """nanovllm/layers/fused_moe.py:218-320,693-787."""

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
                 num_redundant_experts: int = 0, has_bias: bool = False):
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
        if self.scoring_func != "softmax" and not self.use_grouped_topk:
            raise ValueError("Only softmax scoring function is supported for non-grouped topk.")
        self.moe_config = MoEConfig(
            num_experts=self.global_num_experts, experts_per_token=top_k, hidden_dim=hidden_size,
            num_local_experts=self.local_num_experts,
            moe_parallel_config=self.moe_parallel_config, in_dtype=params_dtype,
            quant_dtype=params_dtype, max_num_tokens=256)
        self.quant_method = UnquantizedFusedMoEMethod(self.moe_config)
        self.quant_method.create_weights(
            layer=self, num_experts=self.local_num_experts, hidden_size=hidden_size,
            intermediate_size_per_partition=self.intermediate_size_per_partition,
            params_dtype=params_dtype, has_bias=has_bias)

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
