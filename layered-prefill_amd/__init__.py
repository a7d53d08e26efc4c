"""MI355X (gfx950) fused-MoE expert path: a drop-in for the MoE native ops and
the Triton grouped GEMM of scale-snu/layered-prefill.

    ops        - topk_softmax / moe_align_block_size / silu_and_mul / ... with the
                 out-parameter signatures of the reference's ``nanovllm.ops``
    fused_moe  - moe_align_block_size / fused_topk / fused_experts as in the
                 reference's ``nanovllm/layers/for_moe/fused_moe.py``
    layer      - FusedMoE module as in ``nanovllm/layers/fused_moe.py``
    workloads  - seeded synthetic inputs of the benchmark configurations

Everything computes through libmoe_gfx950.so (hand-written HIP); there is no
CPU or PyTorch fallback.
"""
from . import _lib, ops, fused_moe, layer, loader, schedule, workloads  # noqa: F401
from .fused_moe import (fused_experts, fused_experts_impl, fused_gate_topk, fused_topk,  # noqa: F401
                        fused_topk_experts, moe_align_block_size, quantize_expert_weights,
                        try_get_optimal_moe_config)
from .layer import (FusedMoE, FusedMoEParallelConfig, MoEConfig, UnquantizedFusedMoEMethod,  # noqa: F401
                    Fp8E4M3FusedMoEMethod, GptOssMLP, RMSNorm, SparseMoeBlock)
