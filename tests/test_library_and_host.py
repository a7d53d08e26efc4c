"""CPU-only checks: the C-ABI library loads and exports what include/*.h
declares, argument validation rejects bad calls before touching a GPU, the
host-side mirror of the reference interface behaves, and the workloads are
reproducible.  No kernel is launched here."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "moe_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for must in ("moe_topk_softmax", "moe_align_block_size", "moe_silu_and_mul", "moe_fused_experts",
                 "moe_sum", "moe_last_error", "moe_fused_experts_workspace_bytes"):
        assert must in names


def test_library_exports_every_declared_symbol(moe):
    lib = ctypes.CDLL(moe._lib.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} declared in include/moe_gfx950.h but not exported"
    assert set(_declared_functions()) == set(moe._lib.EXPORTS)
    assert moe._lib.lib().moe_abi_version() == 2


def test_struct_layout_matches_header(moe):
    # field order of the ctypes mirror follows the C struct
    text = open(os.path.join(ROOT, "include", "moe_gfx950.h")).read()
    body = text[text.index("typedef struct MoeFusedExpertsArgs {"):text.index("} MoeFusedExpertsArgs;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    c_fields = []
    for decl in body.split(";"):
        decl = decl.replace("typedef struct MoeFusedExpertsArgs {", "").strip()
        if not decl:
            continue
        names = decl.split(",")
        first = names[0].split()[-1].lstrip("*")
        c_fields.append(first)
        c_fields.extend(n.strip().lstrip("*") for n in names[1:])
    assert c_fields == [f[0] for f in moe._lib.MoeFusedExpertsArgs._fields_]


def test_argument_validation_without_gpu(moe):
    L = moe._lib.lib()
    assert L.moe_topk_softmax(None, None, None, None, 4, 8, 9, 0, None) == -1
    assert b"exceeds num_experts" in L.moe_last_error()
    assert L.moe_topk_softmax(None, None, None, None, 4, 20000, 2, 0, None) == -2
    assert L.moe_align_block_size(None, 0, 10, 2000, 16, None, 0, None, 0, None, None, 0, None) == -2
    assert L.moe_align_block_size(None, 9, 10, 8, 16, None, 0, None, 0, None, None, 0, None) == -1
    assert L.moe_silu_and_mul(None, None, 4, 0, 2, None) == -1
    assert L.moe_fused_experts(None) == -1
    assert L.moe_topk_softmax(None, None, None, None, 0, 8, 2, 0, None) == 0  # empty batch is a no-op
    assert L.moe_align_workspace_bytes(2048, 128) == 0
    assert L.moe_align_workspace_bytes(67584, 128) >= (132 * 128 + 129) * 4
    want = 0
    for rows, cols in ((67584 + 128 * 127, 768), (67584, 2048)):
        want += -(-rows * cols * 2 // 256) * 256
    # + one counter per 256-slot block (one-launch form of the large-tile passes) + XCD range table
    counters = -(-(-(-(67584 + 128 * 127) // 256) * 4) // 256) * 256
    assert L.moe_fused_experts_workspace_bytes(8448, 2048, 768, 128, 8, 128, 2, 2) == want + counters + 256
    # act dtype code 2 = bf16: streaming blocks, then the large tile from 16 rows per expert on
    for m, bm in ((64, 32), (192, 32), (256, 256), (512, 256), (768, 256), (8448, 256)):
        assert L.moe_preferred_block_size(m, 128, 8, 2, 2) == bm
    # e4m3 weights (code 3) quantise the intermediate between the passes: from 32 rows per expert on
    for m, bm in ((256, 32), (384, 32), (512, 256), (8448, 256)):
        assert L.moe_preferred_block_size(m, 128, 8, 2, 3) == bm
    # fp32 (code 0) has no large-tile kernel: the M tile follows the load
    for m, bm in ((256, 32), (768, 64), (2048, 128), (8448, 256)):
        assert L.moe_preferred_block_size(m, 128, 8, 0, 0) == bm


def test_ops_refuse_cpu_tensors(moe):
    ids = torch.zeros(4, 2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        moe.moe_align_block_size(ids, 16, 8)
    x = torch.zeros(4, 8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        moe.fused_topk(x, torch.zeros(4, 8), 2, True)
    with pytest.raises(RuntimeError, match="no CPU path"):
        moe.ops.silu_and_mul(torch.zeros(4, 4), x)


def test_signatures_match_the_reference_interface(moe):
    # nanovllm/layers/for_moe/fused_moe.py:17-19,393-398,422-442
    assert list(inspect.signature(moe.moe_align_block_size).parameters) == ["topk_ids", "block_size", "num_experts"]
    assert list(inspect.signature(moe.fused_topk).parameters) == ["hidden_states", "gating_output", "topk", "renormalize"]
    fe = inspect.signature(moe.fused_experts).parameters
    # the reference's parameters, in its order; what this build adds comes after them, with a default
    assert list(fe)[:21] == ["hidden_states", "w1", "w2", "w1_bias", "w2_bias", "topk_weights", "topk_ids", "inplace",
                             "activation", "apply_router_weight_on_input", "per_channel_quant", "global_num_experts",
                             "expert_map", "w1_scale", "w2_scale", "w1_zp", "w2_zp", "a1_scale", "a2_scale",
                             "block_shape", "allow_deep_gemm"]
    assert list(fe)[21:] == ["weight_layout"] and fe["weight_layout"].default == "plain"
    assert fe["inplace"].default is False and fe["activation"].default == "silu"
    # csrc/ops.cpp:29-31,46-60
    assert list(inspect.signature(moe.ops.topk_softmax).parameters)[:4] == [
        "topk_weights", "topk_indices", "token_expert_indices", "gating_output"]
    assert list(inspect.signature(moe.ops.moe_align_block_size).parameters) == [
        "topk_ids", "num_experts", "block_size", "sorted_token_ids", "experts_ids", "num_tokens_post_pad"]
    assert list(inspect.signature(moe.ops.silu_and_mul).parameters) == ["out", "input"]


def test_fused_moe_module_parameters(moe):
    # nanovllm/layers/fused_moe.py:119-157: w13 [E, 2I, H], w2 [E, H, I] (+ biases)
    layer = moe.FusedMoE(8, 2, 256, 128, params_dtype=torch.bfloat16, has_bias=True)
    assert tuple(layer.w13_weight.shape) == (8, 256, 256) and layer.w13_weight.dtype == torch.bfloat16
    assert tuple(layer.w2_weight.shape) == (8, 256, 128)
    assert tuple(layer.w13_bias.shape) == (8, 256) and tuple(layer.w2_bias.shape) == (8, 256)
    assert not layer.w13_weight.requires_grad
    assert layer.tp_size == 1 and layer.tp_rank == 0 and layer.renormalize and layer.activation == "silu"
    with pytest.raises(ValueError, match="Only softmax"):
        moe.FusedMoE(8, 2, 256, 128, scoring_func="sigmoid")


def test_fused_experts_shape_assertions(moe):
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    w1 = torch.zeros(2, 32, 48, dtype=torch.bfloat16)
    w2 = torch.zeros(2, 64, 16, dtype=torch.bfloat16)
    tw = torch.zeros(4, 2)
    ids = torch.zeros(4, 2, dtype=torch.int32)
    with pytest.raises(AssertionError, match="Hidden size mismatch"):
        moe.fused_experts(x, w1, w2, None, None, tw, ids)
    w1 = torch.zeros(2, 32, 64, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="topk shape mismatch"):
        moe.fused_experts(x, w1, w2, None, None, tw[:, :1], ids)
    with pytest.raises(ValueError, match="Unsupported FusedMoe activation"):
        moe.fused_experts(x, w1, w2, None, None, tw, ids, activation="relu")


def test_fused_experts_takes_ragged_sizes_except_with_e4m3(moe):
    """The reference's Triton kernel masks ragged K and N (for_moe/fused_moe.py:191-205,218-223).
    So does this build for 16-bit and fp32 weights (an element-by-element kernel): such calls pass
    every host check and stop at the device check here.  e4m3 rows move in 16-byte chunks only."""
    tw = torch.zeros(4, 2)
    ids = torch.zeros(4, 2, dtype=torch.int32)
    x = torch.zeros(4, 60, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):           # H = 60
        moe.fused_experts(x, torch.zeros(2, 32, 60, dtype=torch.bfloat16), torch.zeros(2, 60, 16, dtype=torch.bfloat16),
                          None, None, tw, ids)
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):           # I = 12
        moe.fused_experts(x, torch.zeros(2, 24, 64, dtype=torch.bfloat16), torch.zeros(2, 64, 12, dtype=torch.bfloat16),
                          None, None, tw, ids)
    w1 = torch.zeros(2, 32, 68, dtype=torch.bfloat16)[:, :, :64]      # row stride 68
    with pytest.raises(RuntimeError, match="no CPU path"):
        moe.fused_experts(x, w1, torch.zeros(2, 64, 16, dtype=torch.bfloat16), None, None, tw, ids)
    with pytest.raises(RuntimeError, match="no CPU path"):           # fp32, H = 62
        moe.fused_experts(torch.zeros(4, 62), torch.zeros(2, 24, 62), torch.zeros(2, 62, 12), None, None, tw, ids)
    # e4m3: multiples of 16 elements
    f8 = torch.float8_e4m3fn
    with pytest.raises(AssertionError, match="multiples of 16"):
        moe.fused_experts(torch.zeros(4, 72, dtype=torch.bfloat16), torch.zeros(2, 32, 72).to(f8), torch.zeros(2, 72, 16).to(f8),
                          None, None, tw, ids, per_channel_quant=True, w1_scale=torch.ones(2, 32), w2_scale=torch.ones(2, 72))
    # the stride of a dimension of size 1 says nothing: one expert cut out of a larger tensor
    one13 = torch.zeros(3, 32, 64, dtype=torch.bfloat16).as_strided((1, 32, 64), (2051, 64, 1))
    one2 = torch.zeros(3, 64, 16, dtype=torch.bfloat16)[:1]
    with pytest.raises(RuntimeError, match="no CPU path"):
        moe.fused_experts(x, one13, one2, None, None, tw, torch.zeros(4, 2, dtype=torch.int32))
    with pytest.raises(AssertionError, match="global_num_experts"):
        moe.fused_experts(x, torch.zeros(2, 32, 64, dtype=torch.bfloat16), torch.zeros(2, 64, 16, dtype=torch.bfloat16),
                          None, None, tw, ids, global_num_experts=4)
    with pytest.raises(RuntimeError, match="no CPU path"):           # and only then the device check
        moe.fused_experts(x, torch.zeros(2, 32, 64, dtype=torch.bfloat16), torch.zeros(2, 64, 16, dtype=torch.bfloat16),
                          None, None, tw, ids)


def test_block_size_rule_follows_the_activation_dtype(moe):
    cfg = moe.fused_moe.try_get_optimal_moe_config
    w1, w2 = (128, 1536, 2048), (128, 2048, 768)
    assert cfg(w1, w2, 8, None, 768, act_dtype=torch.bfloat16)["BLOCK_SIZE_M"] == 256
    assert cfg(w1, w2, 8, None, 768, act_dtype=torch.float16)["BLOCK_SIZE_M"] == 256
    assert cfg(w1, w2, 8, None, 768, act_dtype=torch.float32)["BLOCK_SIZE_M"] == 64    # fp32 has its own rule
    assert cfg(w1, w2, 8, None, 2048, act_dtype=torch.float32)["BLOCK_SIZE_M"] == 128
    assert cfg(w1, w2, 8, "fp8_w8a8", 384)["BLOCK_SIZE_M"] == 32


def test_plan_and_counters_lie_inside_the_workspace_behind_the_data(moe):
    """Every region of a moe_fused_experts workspace is laid out from
    T*K + E*(block-1), never from the length of the caller's sorted_token_ids buffer:
    the per-block counters and the range table sit behind the intermediates."""
    L = moe._lib.lib()
    for T, H, I, E, K, bs, act, wgt in ((8448, 2048, 768, 128, 8, 256, 2, 2), (256, 2048, 768, 128, 8, 256, 2, 2),
                                        (1, 64, 64, 4, 1, 256, 1, 1), (3000, 512, 256, 16, 4, 512, 2, 3),
                                        (777, 128, 96, 8, 2, 256, 2, 3)):
        total = L.moe_fused_experts_workspace_bytes(T, H, I, E, K, bs, act, wgt)
        b, d = ctypes.c_int64(), ctypes.c_int64()
        n, cap = ctypes.c_int32(), ctypes.c_int32()
        assert L.moe_fused_experts_plan_layout(T, H, I, E, K, bs, act, wgt, ctypes.byref(b), ctypes.byref(d),
                                               ctypes.byref(n), ctypes.byref(cap)) == 1
        sorted_cap = T * K + E * (bs - 1)
        rows = -(-sorted_cap // bs) * bs
        up = lambda v: -(-v // 256) * 256
        data = up(rows * I * 2) + up(T * K * H * 2)
        if wgt == 3:
            data += up(T * H) + up(T * 4) + up(rows * I) + up(rows * 4)
        assert n.value == -(-sorted_cap // 256) and 1 <= cap.value <= n.value
        assert d.value >= data and d.value + 4 * n.value <= b.value and b.value + 256 == total
    # blocks that are not multiples of 256, or fp32, have no plan
    assert L.moe_fused_experts_plan_layout(256, 2048, 768, 128, 8, 32, 2, 2, ctypes.byref(b), ctypes.byref(d),
                                           ctypes.byref(n), ctypes.byref(cap)) == 0
    assert L.moe_fused_experts_plan_layout(256, 2048, 768, 128, 8, 256, 0, 0, ctypes.byref(b), ctypes.byref(d),
                                           ctypes.byref(n), ctypes.byref(cap)) == 0


def test_workloads_are_reproducible_and_skewed(moe):
    wl = moe.workloads
    a = wl.make_inputs(wl.QWEN3_30B_A3B, 256, 1, torch.bfloat16)
    b = wl.make_inputs(wl.QWEN3_30B_A3B, 256, 1, torch.bfloat16)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert a[0].shape == (256, 2048) and a[1].shape == (256, 128) and a[1].dtype == torch.float32
    bias = wl.zipf_bias(128, torch.Generator().manual_seed(3))
    assert abs(bias.mean().item()) < 1e-5 and bias.max() - bias.min() > 4.0
    assert wl.layer_flops(8448, wl.QWEN3_30B_A3B) == 637802643456
    assert wl.layer_flops(256, wl.QWEN3_30B_A3B) == 19327352832
    assert wl.layer_bytes(256, wl.QWEN3_30B_A3B, 128) == 1207959552 + 2 * 1048576 + 131072
    shape, x, logits, w13, w2 = wl.make_config("tiny_fp32")
    assert w13.shape == (8, 256, 256) and w2.shape == (8, 256, 128) and x.dtype == torch.float32


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "layered-prefill_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "__init__.py" and False, f
