"""Checkpoint loading into FusedMoE (CPU): the placement rules of the
reference's loader (nanovllm/layers/fused_moe.py:330-658,789-821 and
nanovllm/utils/loader.py:37-93), checked against tensors assembled by hand."""
import os

import pytest
import torch


def _ckpt(E, H, I, dtype=torch.float32, layer=3, bias=False):
    g = torch.Generator().manual_seed(5)
    t = {}
    for e in range(E):
        p = f"model.layers.{layer}.mlp.experts.{e}."
        t[p + "gate_proj.weight"] = torch.randn(I, H, generator=g).to(dtype)
        t[p + "up_proj.weight"] = torch.randn(I, H, generator=g).to(dtype)
        t[p + "down_proj.weight"] = torch.randn(H, I, generator=g).to(dtype)
    if bias:
        p = f"model.layers.{layer}.mlp.experts."
        t[p + "gate_up_proj_bias"] = torch.randn(E, 2 * I, generator=g).to(dtype)
        t[p + "down_proj_bias"] = torch.randn(E, H, generator=g).to(dtype)
    t[f"model.layers.{layer}.mlp.gate.weight"] = torch.randn(E, H, generator=g).to(dtype)
    return t


def test_expert_params_mapping_known_answer(moe):
    # nanovllm/layers/fused_moe.py:789-821: per physical expert w1, w2, w3 in this order;
    # the redundant expert (physical id 2) replays logical expert 0
    got = moe.FusedMoE.make_expert_params_mapping("gate_proj", "down_proj", "up_proj", 2, 1)
    assert got == [
        ("experts.w13_", "experts.0.gate_proj.", 0, "w1"),
        ("experts.w2_", "experts.0.down_proj.", 0, "w2"),
        ("experts.w13_", "experts.0.up_proj.", 0, "w3"),
        ("experts.w13_", "experts.1.gate_proj.", 1, "w1"),
        ("experts.w2_", "experts.1.down_proj.", 1, "w2"),
        ("experts.w13_", "experts.1.up_proj.", 1, "w3"),
        ("experts.w13_", "experts.0.gate_proj.", 2, "w1"),
        ("experts.w2_", "experts.0.down_proj.", 2, "w2"),
        ("experts.w13_", "experts.0.up_proj.", 2, "w3"),
    ]


def test_loader_places_gate_up_down(moe):
    E, H, I = 4, 32, 24
    ck = _ckpt(E, H, I)
    layer = moe.FusedMoE(E, 2, H, I, params_dtype=torch.float32)
    layer.w13_weight.data.fill_(float("nan"))
    layer.w2_weight.data.fill_(float("nan"))
    rest = moe.loader.load_moe_experts(lambda idx: layer if idx == 3 else None, ck.items())
    assert rest == ["model.layers.3.mlp.gate.weight"]
    for e in range(E):
        p = f"model.layers.3.mlp.experts.{e}."
        # gate rows [0, I), up rows [I, 2I): what silu(first half) * second half expects
        assert torch.equal(layer.w13_weight.data[e, :I], ck[p + "gate_proj.weight"])
        assert torch.equal(layer.w13_weight.data[e, I:], ck[p + "up_proj.weight"])
        assert torch.equal(layer.w2_weight.data[e], ck[p + "down_proj.weight"])
    assert hasattr(layer.w13_weight, "weight_loader")


def test_loader_slices_for_a_tensor_parallel_rank(moe, monkeypatch):
    E, H, I, tp = 2, 16, 24, 2
    ck = _ckpt(E, H, I, bias=True)
    for rank in range(tp):
        monkeypatch.setattr(moe.layer.FusedMoEParallelConfig, "make",
                            staticmethod(lambda r=rank: moe.layer.FusedMoEParallelConfig(tp, r)))
        layer = moe.FusedMoE(E, 2, H, I, params_dtype=torch.float32, has_bias=True)
        Ip = I // tp
        assert tuple(layer.w13_weight.shape) == (E, 2 * Ip, H) and tuple(layer.w2_weight.shape) == (E, H, Ip)
        moe.loader.load_moe_experts(lambda idx: layer, ck.items())
        for e in range(E):
            p = f"model.layers.3.mlp.experts.{e}."
            sl = slice(rank * Ip, (rank + 1) * Ip)
            # column-parallel gate/up: this rank's rows; row-parallel down: its columns
            assert torch.equal(layer.w13_weight.data[e, :Ip], ck[p + "gate_proj.weight"][sl])
            assert torch.equal(layer.w13_weight.data[e, Ip:], ck[p + "up_proj.weight"][sl])
            assert torch.equal(layer.w2_weight.data[e], ck[p + "down_proj.weight"][:, sl])
        gu = ck["model.layers.3.mlp.experts.gate_up_proj_bias"]
        assert torch.equal(layer.w13_bias.data, gu[:, rank * 2 * Ip:(rank + 1) * 2 * Ip])
        down = ck["model.layers.3.mlp.experts.down_proj_bias"]
        assert torch.equal(layer.w2_bias.data, down if rank == 0 else torch.zeros_like(down))


def test_loader_reads_a_safetensors_directory(moe, tmp_path):
    from safetensors.torch import save_file
    E, H, I = 3, 16, 8
    ck = _ckpt(E, H, I, dtype=torch.bfloat16)
    names = sorted(ck)
    save_file({k: ck[k] for k in names[:5]}, os.path.join(tmp_path, "model-00001.safetensors"))
    save_file({k: ck[k] for k in names[5:]}, os.path.join(tmp_path, "model-00002.safetensors"))
    layer = moe.FusedMoE(E, 2, H, I, params_dtype=torch.bfloat16)
    rest = moe.loader.load_moe_experts(lambda idx: layer, moe.loader.iter_safetensors(str(tmp_path)))
    assert rest == ["model.layers.3.mlp.gate.weight"]
    assert torch.equal(layer.w13_weight.data[2, I:], ck["model.layers.3.mlp.experts.2.up_proj.weight"])


def test_loader_all_experts_in_one_tensor_and_errors(moe):
    E, H, I = 2, 8, 8
    layer = moe.FusedMoE(E, 1, H, I, params_dtype=torch.float32, has_bias=True)
    w = torch.arange(E * 2 * I * H, dtype=torch.float32).reshape(E, 2 * I, H)
    layer.weight_loader(layer.w13_weight, w, "experts.gate_up_proj.weight", "all", 0)
    assert torch.equal(layer.w13_weight.data, w)
    assert layer.weight_loader(layer.w2_weight, torch.ones(H, I), "experts.0.down_proj.weight", "w2", 1,
                               return_success=True) is True
    assert torch.equal(layer.w2_weight.data[1], torch.ones(H, I))
    with pytest.raises(ValueError, match="shard_id must be"):
        layer.weight_loader(layer.w2_weight, torch.ones(H, I), "experts.0.down_proj.weight", "w7", 0)
    with pytest.raises(ValueError, match="g_idx"):
        layer.weight_loader(layer.w2_weight, torch.ones(H), "experts.0.down_proj.g_idx", "w2", 0)
    with pytest.raises(NotImplementedError, match="MX-FP4"):
        moe.loader.load_expert_tensor(lambda i: layer, "model.layers.0.mlp.experts.down_proj_blocks",
                                      torch.zeros(1))


@pytest.mark.gpu
def test_loaded_fp8_layer_matches_the_fp8_oracle(moe, oracle, dev):
    """Checkpoint -> loader -> one-time e4m3 quantisation -> forward, against the
    oracle fed with the same checkpoint tensors."""
    E, H, I, T, K = 8, 256, 128, 96, 2
    ck = {k: v * 0.05 for k, v in _ckpt(E, H, I, dtype=torch.bfloat16).items()}
    layer = moe.FusedMoE(E, K, H, I, params_dtype=torch.bfloat16, quantization="fp8_e4m3")
    moe.loader.load_moe_experts(lambda idx: layer, ck.items())
    w13 = layer.w13_weight.data.clone()
    w2 = layer.w2_weight.data.clone()
    layer.to(dev)
    layer.process_weights_after_loading()
    assert layer.w13_weight.dtype == torch.float8_e4m3fn and tuple(layer.w13_weight_scale.shape) == (E, 2 * I)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    out = layer(x.to(dev).clone(), logits.to(dev))
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    q13, s13 = oracle.quant_weight_per_channel(w13)
    q2, s2 = oracle.quant_weight_per_channel(w2)
    ref = oracle.fused_experts_fp8_ref(x, q13, s13, q2, s2, tw, ids, mirror_rounding=True)
    got = out.float().cpu()
    assert (got - ref).abs().max() <= 0.03 * ref.abs().max() + 2e-2 * ref.abs().max()
