"""GPU parity of the expert MLP (grouped GEMMs, fused activation, combine) and
of the stand-alone activation / combine ops against the CPU oracle."""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

# tolerances of the north star: bf16 results against the fp32 oracle
RTOL, ATOL = 2e-2, 1e-2


def _layer(E, H, I, T, K, seed, dtype, wstd=0.05):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(dtype)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * wstd).to(dtype)
    w2 = (torch.randn(E, H, I, generator=g) * wstd).to(dtype)
    logits = torch.randn(T, E, generator=g)
    return x, w13, w2, logits


def _close(got, want, rtol=RTOL, atol=ATOL):
    got, want = got.float().cpu(), want.float()
    bad = (got - want).abs() > atol + rtol * want.abs()
    assert not bad.any(), f"{bad.sum().item()} of {bad.numel()} off; max abs err {(got - want).abs().max().item():.4g}"


def _mode(moe, T, E, K, H, dtype, fp8=False, bm=None, activation="silu"):
    """The rounding definition of the kernel the library picks for this call.  The
    large-tile kernel (alignment blocks that are multiples of 256 slots, reduction
    length of the gate-up pass a multiple of its K tile: 64 elements of 16 bits, 128
    of e4m3) forms silu(gate) * up on its fp32 accumulators and rounds the
    intermediate once (``mirror_rounding="fused"``); every other kernel, and the
    large-tile kernel with the other activations, rounds at every store the
    reference has (``True``)."""
    if bm is None:
        bm = moe.fused_moe.try_get_optimal_moe_config(
            (E, 0, H), (E, H, 0), K, "fp8_w8a8" if fp8 else None, min(T, 65536), act_dtype=dtype)["BLOCK_SIZE_M"]
    large = bm % 256 == 0 and H % (128 if fp8 else 64) == 0 and dtype != torch.float32
    return "fused" if large and activation == "silu" else True


def _close_mirrored(got, ref_fn, mode, **tol):
    """Against the oracle that rounds where the kernel that ran stores (``_mode``)."""
    assert mode is True or mode == "fused"
    _close(got, ref_fn(mode), **tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("E,H,I,T,K", [(8, 256, 128, 64, 2), (4, 64, 64, 1, 1), (16, 512, 192, 300, 4),
                                       (8, 128, 96, 777, 2), (128, 512, 256, 256, 8),
                                       (3, 72, 40, 50, 2)])
def test_fused_experts_against_oracle(moe, oracle, dev, dtype, E, H, I, T, K):
    print(f"fused_experts {dtype} E={E} H={H} I={I} T={T} K={K}", flush=True)
    x, w13, w2, logits = _layer(E, H, I, T, K, 17 + E + T, dtype)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    out = moe.fused_experts(x.to(dev), w13.to(dev), w2.to(dev), None, None, tw.to(dev), ids.to(dev))
    torch.cuda.synchronize()
    assert out.dtype == dtype and out.shape == x.shape
    _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids))
    # against the oracle that rounds where the reference stores intermediates the
    # agreement is much tighter (only the fp32 summation order differs)
    _close_mirrored(out, lambda m: oracle.fused_experts_ref(x, w13, w2, tw, ids, mirror_rounding=m),
                    _mode(moe, T, E, K, H, dtype), rtol=1.6e-2, atol=2e-3)


@pytest.mark.parametrize("E,H,I,T,K", [(8, 256, 128, 64, 2), (16, 512, 192, 300, 4), (3, 72, 40, 50, 2),
                                       (3, 68, 36, 50, 2)])   # the last: multiples of 4 elements (16 bytes of fp32) only
def test_fused_experts_fp32_against_oracle(moe, oracle, dev, E, H, I, T, K):
    """fp32 activations and weights (the reference accepts them,
    nanovllm/layers/for_moe/fused_moe.py:491-493): fp32 MFMA, no rounding points,
    so only the summation order separates the result from the fp32 oracle."""
    x, w13, w2, logits = _layer(E, H, I, T, K, 7 + E + T, torch.float32)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    out = moe.fused_experts(x.to(dev), w13.to(dev), w2.to(dev), None, None, tw.to(dev), ids.to(dev))
    assert out.dtype == torch.float32
    _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("bm", [32, 64, 96, 128, 256, 512])
def test_every_block_size_kernel(moe, oracle, dev, bm, monkeypatch):
    x, w13, w2, logits = _layer(16, 256, 128, 500, 4, 5, torch.bfloat16)
    tw, ids, _ = oracle.topk_softmax(logits, 4, renormalize=True)
    monkeypatch.setattr(moe.fused_moe, "try_get_optimal_moe_config",
                        lambda *a, **k: {"BLOCK_SIZE_M": bm})
    out = moe.fused_experts(x.to(dev), w13.to(dev), w2.to(dev), None, None, tw.to(dev), ids.to(dev))
    _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids))


def test_inplace_aliases_input_and_matches(moe, oracle, dev):
    x, w13, w2, logits = _layer(8, 256, 128, 200, 2, 9, torch.bfloat16)
    tw, ids, _ = oracle.topk_softmax(logits, 2, renormalize=True)
    xd = x.to(dev)
    ref = moe.fused_experts(xd.clone(), w13.to(dev), w2.to(dev), None, None, tw.to(dev), ids.to(dev))
    out = moe.fused_experts(xd, w13.to(dev), w2.to(dev), None, None, tw.to(dev), ids.to(dev), inplace=True)
    assert out.data_ptr() == xd.data_ptr()
    assert torch.equal(out, ref)


def test_bias_router_weight_on_input_and_other_activations(moe, oracle, dev):
    E, H, I, T, K = 8, 128, 64, 150, 1
    x, w13, w2, logits = _layer(E, H, I, T, K, 21, torch.bfloat16)
    g = torch.Generator().manual_seed(2)
    b13 = (torch.randn(E, 2 * I, generator=g) * 0.1).bfloat16()
    b2 = (torch.randn(E, H, generator=g) * 0.1).bfloat16()
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=False)
    d = lambda t: t.to(dev)
    for act in ("silu", "swigluoai", "gelu"):
        for on_input in (False, True):
            out = moe.fused_experts(d(x), d(w13), d(w2), d(b13), d(b2), d(tw), d(ids), activation=act,
                                    apply_router_weight_on_input=on_input)
            _close_mirrored(out, lambda m: oracle.fused_experts_ref(
                x, w13, w2, tw, ids, activation=act, w1_bias=b13, w2_bias=b2,
                apply_router_weight_on_input=on_input, mirror_rounding=m),
                _mode(moe, T, E, K, H, torch.bfloat16, activation=act), rtol=2e-2, atol=4e-3)
            # and the north-star bound against the oracle that rounds nowhere
            _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids, activation=act, w1_bias=b13, w2_bias=b2,
                                                 apply_router_weight_on_input=on_input))
    with pytest.raises(ValueError, match="Unsupported FusedMoe activation"):
        moe.fused_experts(d(x), d(w13), d(w2), None, None, d(tw), d(ids), activation="relu")


def test_strided_expert_weights(moe, oracle, dev):
    # w13 / w2 as views with a padded row stride (last dimension contiguous)
    E, H, I, T, K = 4, 128, 64, 90, 2
    x, w13, w2, logits = _layer(E, H, I, T, K, 33, torch.bfloat16)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    big13 = torch.zeros(E, 2 * I, H + 64, dtype=torch.bfloat16, device=dev)
    big13[:, :, :H] = w13.to(dev)
    big2 = torch.zeros(E, H, I + 8, dtype=torch.bfloat16, device=dev)
    big2[:, :, :I] = w2.to(dev)
    out = moe.fused_experts(x.to(dev), big13[:, :, :H], big2[:, :, :I], None, None, tw.to(dev), ids.to(dev))
    _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids))


def test_linearity_and_permutation_properties_at_full_decode_size(moe, oracle, dev):
    """Config 2 (256 decode tokens): every row against the fp32 oracle and against the
    oracle that rounds where the kernel stores, plus the size-independent properties."""
    wl = moe.workloads
    shape, x, logits, w13, w2 = wl.make_config("decode_256")
    d = lambda t: t.to(dev)
    tw, ids, _ = moe.fused_topk(d(x), d(logits), shape.top_k, True)
    a = moe.fused_experts(d(x), d(w13), d(w2), None, None, tw, ids)
    perm = torch.randperm(x.shape[0], generator=torch.Generator().manual_seed(0)).to(dev)
    b = moe.fused_experts(d(x)[perm].contiguous(), d(w13), d(w2), None, None, tw[perm].contiguous(),
                          ids[perm].contiguous())
    _close(b, a[perm].cpu(), rtol=1e-2, atol=2e-3)
    z = moe.fused_experts(d(x), d(w13), d(w2), None, None, torch.zeros_like(tw), ids)
    assert torch.count_nonzero(z) == 0
    _close(a, oracle.fused_experts_ref(x, w13, w2, tw.cpu(), ids.cpu()))
    mode = _mode(moe, x.shape[0], shape.experts, shape.top_k, shape.hidden, torch.bfloat16)
    _close(a, oracle.fused_experts_ref(x, w13, w2, tw.cpu(), ids.cpu(), mirror_rounding=mode), rtol=1.6e-2, atol=2e-3)


def test_layered_prefill_batch_every_row(moe, oracle, dev):
    """Config 3 (8192 prefill + 256 decode tokens): all 8448 rows against the fp32
    oracle at the north-star tolerance and, tightly, against the oracle that rounds
    where the large-tile kernel stores.  Config 4: each of the 16 chunks (512 prefill
    rows + the 256 decode rows) gives the rows of the single pass."""
    wl = moe.workloads
    shape, x, logits, w13, w2 = wl.make_config("layered_8192p_256d")
    d = lambda t: t.to(dev)
    w13d, w2d = d(w13), d(w2)
    tw, ids, _ = moe.fused_topk(d(x), d(logits), shape.top_k, True)
    out = moe.fused_experts(d(x), w13d, w2d, None, None, tw, ids)
    torch.cuda.synchronize()
    _close(out, oracle.fused_experts_ref(x, w13, w2, tw.cpu(), ids.cpu()))
    mode = _mode(moe, x.shape[0], shape.experts, shape.top_k, shape.hidden, torch.bfloat16)
    assert mode == "fused"
    _close(out, oracle.fused_experts_ref(x, w13, w2, tw.cpu(), ids.cpu(), mirror_rounding=mode), rtol=1.6e-2, atol=2e-3)
    # chunked prefill (16 x (512 + 256)) gives the same rows as the single pass
    outc = out.cpu()
    for c in range(16):
        sel = torch.cat([torch.arange(c * 512, (c + 1) * 512), torch.arange(8192, 8448)]).to(dev)
        part = moe.fused_experts(d(x)[sel].contiguous(), w13d, w2d, None, None, tw[sel].contiguous(),
                                 ids[sel].contiguous())
        _close(part, outc[sel.cpu()], rtol=1e-2, atol=2e-3)


def test_fused_moe_module_forward(moe, oracle, dev):
    wl = moe.workloads
    shape, x, logits, w13, w2 = wl.make_config("tiny_fp32")
    layer = moe.FusedMoE(shape.experts, shape.top_k, shape.hidden, shape.intermediate,
                         params_dtype=torch.bfloat16, renormalize=True).to(dev)
    assert tuple(layer.w13_weight.shape) == (8, 256, 256) and tuple(layer.w2_weight.shape) == (8, 256, 128)
    layer.w13_weight.data.copy_(w13)
    layer.w2_weight.data.copy_(w2)
    xb = x.bfloat16()
    hs = xb.to(dev)
    out = layer(hs, logits.to(dev))
    assert out.data_ptr() == hs.data_ptr()  # inplace=True, as the reference's apply()
    tw, ids, _ = oracle.fused_topk(xb, logits, shape.top_k, True)
    ref = oracle.fused_experts_ref(xb, w13.bfloat16(), w2.bfloat16(), tw, ids)
    _close(out, ref)


# ------------------------------------------------------------------ element-wise ops
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,d", [(1, 8), (5, 768), (300, 96), (17, 7)])
def test_silu_and_mul_bit_exact(moe, oracle, dev, dtype, rows, d):
    x = (torch.randn(rows, 2 * d, generator=torch.Generator().manual_seed(rows + d)) * 4).to(dtype)
    out = torch.empty(rows, d, dtype=dtype, device=dev)
    moe.ops.silu_and_mul(out, x.to(dev))
    want = oracle.silu_and_mul(x)
    assert torch.equal(out.cpu().view(torch.int16 if dtype != torch.float32 else torch.int32),
                       want.view(torch.int16 if dtype != torch.float32 else torch.int32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,d", [(40, 360), (5000, 7), (3000, 1)])
def test_swigluoai_and_mul_bit_exact(moe, oracle, dev, dtype, rows, d):
    """Vector path (d a multiple of 8) and element path.  fp16 with many rows is the case in
    which a multiplication folded into the narrowing conversion (one rounding instead of
    two) shows: about one element in ten thousand."""
    x = (torch.randn(rows, 2 * d, generator=torch.Generator().manual_seed(1)) * 3).to(dtype)
    out = torch.empty(rows, d, dtype=dtype, device=dev)
    moe.ops.swigluoai_and_mul(out, x.to(dev), 1.702, 7.0)
    want = oracle.swigluoai_and_mul(x, 1.702, 7.0)
    assert torch.equal(out.cpu().view(torch.int16 if dtype != torch.float32 else torch.int32),
                       want.view(torch.int16 if dtype != torch.float32 else torch.int32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_moe_sum(moe, dev, dtype):
    x = torch.randn(33, 8, 200, generator=torch.Generator().manual_seed(3)).to(dtype)
    out = torch.empty(33, 200, dtype=dtype, device=dev)
    moe.ops.moe_sum(x.to(dev), out)
    want = x.float().sum(1)
    assert torch.allclose(out.cpu().float(), want, rtol=2 ** -7 if dtype != torch.float32 else 1e-6, atol=1e-5)


def test_quant_rows_e4m3_matches_oracle(moe, oracle, dev):
    w = torch.randn(64, 512, generator=torch.Generator().manual_seed(7)) * 0.02
    w[3] = 0
    w[5] = 0
    w[5, 9], w[5, 200] = 1e-38, -3e-39          # 1 / (amax / 448) would overflow: the scale is floored
    w[6] *= 2.0 ** -95                           # rows around the floor of 2^-100
    w[7] *= 2.0 ** -105
    for dtype in (torch.float32, torch.bfloat16):
        wd = w.to(dtype)
        q, s = moe.ops.quant_rows_e4m3(wd.to(dev))
        oq, os_ = oracle.quant_weight_per_channel(wd[None])
        assert torch.equal(s.cpu(), os_[0])
        assert torch.equal(q.cpu(), oq[0])
        assert not ((q.cpu() & 0x7f) == 0x7f).any() and s.cpu()[5] == 2.0 ** -100


# ------------------------------------------------------------------ fp8 e4m3 variant
def _close_fp8(got, want, atol=1e-2):
    # north star: rtol 6e-2 against the fp32 dequantised oracle (atol 1e-2 as for bf16)
    _close(got, want, rtol=6e-2, atol=atol)


@pytest.mark.parametrize("E,H,I,T,K", [(8, 256, 128, 64, 2), (16, 512, 256, 300, 4), (128, 512, 256, 256, 8),
                                       (4, 144, 48, 33, 2)])
def test_fused_experts_fp8_against_dequantised_oracle(moe, oracle, dev, E, H, I, T, K):
    print(f"fused_experts fp8 E={E} H={H} I={I} T={T} K={K}", flush=True)
    x, w13, w2, logits = _layer(E, H, I, T, K, 91 + E + T, torch.bfloat16)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    w13q, w13s, w2q, w2s = moe.quantize_expert_weights(w13.to(dev), w2.to(dev))
    # the GPU quantiser is the oracle's, bit for bit
    oq13, os13 = oracle.quant_weight_per_channel(w13)
    oq2, os2 = oracle.quant_weight_per_channel(w2)
    assert torch.equal(w13q.view(torch.uint8).cpu(), oq13) and torch.equal(w13s.cpu(), os13)
    assert torch.equal(w2q.view(torch.uint8).cpu(), oq2) and torch.equal(w2s.cpu(), os2)
    out = moe.fused_experts(x.to(dev), w13q, w2q, None, None, tw.to(dev), ids.to(dev),
                            per_channel_quant=True, w1_scale=w13s, w2_scale=w2s)
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16
    # (a) the oracle that rounds where the kernels store 16-bit intermediates: tight
    _close_mirrored(out, lambda m: oracle.fused_experts_fp8_ref(x, oq13, os13, oq2, os2, tw, ids, mirror_rounding=m),
                    _mode(moe, T, E, K, H, torch.bfloat16, fp8=True), rtol=2e-2,
                    atol=0.03 * out.float().abs().max().item())
    # (b) the pure fp32 dequantised oracle.  These small layers use 2.5x larger weights
    # than the benchmark layer, so the absolute floor is stated relative to the output
    # scale: one e4m3 step (2^-3 relative) of a typical element.  Re-quantising the
    # 16-bit intermediate instead of its fp32 value flips some e4m3 roundings; the
    # resulting difference is ~4x below the e4m3 noise of the oracle itself.
    ref = oracle.fused_experts_fp8_ref(x, oq13, os13, oq2, os2, tw, ids)
    _close_fp8(out, ref, atol=0.125 * ref.float().pow(2).mean().sqrt().item() * 1.5)
    # and it stays near the unquantised layer (loose sanity bound)
    full = oracle.fused_experts_ref(x, w13, w2, tw, ids)
    assert (out.float().cpu() - full).abs().max() < 0.25 * full.abs().max() + 0.05


@pytest.mark.parametrize("bm", [32, 64, 128, 256, 512])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp8_every_block_size_kernel(moe, oracle, dev, bm, dtype, monkeypatch):
    """Blocks of 256 slots run the large-tile e4m3 kernel (K = 64 MFMA steps),
    smaller ones the register-staged kernels; both must agree with the oracle
    that rounds where the kernels store."""
    x, w13, w2, logits = _layer(16, 512, 256, 700, 4, 77, dtype)
    tw, ids, _ = oracle.topk_softmax(logits, 4, renormalize=True)
    w13q, w13s, w2q, w2s = moe.quantize_expert_weights(w13.to(dev), w2.to(dev))
    monkeypatch.setattr(moe.fused_moe, "try_get_optimal_moe_config",
                        lambda *a, **k: {"BLOCK_SIZE_M": bm})
    out = moe.fused_experts(x.to(dev), w13q, w2q, None, None, tw.to(dev), ids.to(dev),
                            per_channel_quant=True, w1_scale=w13s, w2_scale=w2s)
    torch.cuda.synchronize()
    _close_mirrored(out, lambda m: oracle.fused_experts_fp8_ref(
        x, w13q.view(torch.uint8).cpu(), w13s.cpu(), w2q.view(torch.uint8).cpu(), w2s.cpu(), tw, ids,
        mirror_rounding=m), _mode(moe, 700, 16, 4, 512, dtype, fp8=True, bm=bm), rtol=2e-2,
        atol=0.03 * out.float().abs().max().item())


def test_fp8_layered_prefill_batch_every_row(moe, oracle, dev):
    """Config 5: the 8192+256 batch with e4m3 weights and per-token e4m3
    activations, against the fp32 dequantised oracle and the one that rounds where the
    kernels store."""
    wl = moe.workloads
    shape, x, logits, w13, w2 = wl.make_config("layered_8192p_256d")
    d = lambda t: t.to(dev)
    w13q, w13s, w2q, w2s = moe.quantize_expert_weights(d(w13), d(w2))
    tw, ids, _ = moe.fused_topk(d(x), d(logits), shape.top_k, True)
    out = moe.fused_experts(d(x), w13q, w2q, None, None, tw, ids, per_channel_quant=True,
                            w1_scale=w13s, w2_scale=w2s)
    torch.cuda.synchronize()
    rows = torch.arange(x.shape[0])   # all 8448
    q13, q2 = w13q.view(torch.uint8).cpu(), w2q.view(torch.uint8).cpu()
    ref = oracle.fused_experts_fp8_ref(x[rows], q13, w13s.cpu(), q2, w2s.cpu(), tw.cpu()[rows], ids.cpu()[rows])
    # The kernels quantise the stored 16-bit intermediate, this oracle its fp32 value: an element
    # that the 16-bit rounding (or the row scale derived from it) moves across an e4m3 tie changes
    # by a whole e4m3 step, about one element in sixty.  Over the 17.3 million outputs of the whole
    # batch the tail of those flips reaches 0.025 (12 elements beyond 0.017), so: rtol 6e-2 with the
    # absolute floor at one and a half e4m3 steps (1.5 x 2^-3) of a typical output for every
    # element, and the bf16 floor of 1e-2 for all but 1 in 10 000.
    got = out[rows.to(dev)].float().cpu()
    _close_fp8(got, ref, atol=0.1875 * ref.pow(2).mean().sqrt().item())
    off = (got - ref).abs() > 1e-2 + 6e-2 * ref.abs()
    assert off.float().mean().item() <= 1e-4, f"{off.sum().item()} of {off.numel()} beyond rtol 6e-2 / atol 1e-2"
    mode = _mode(moe, x.shape[0], shape.experts, shape.top_k, shape.hidden, torch.bfloat16, fp8=True)
    assert mode == "fused"
    refm = oracle.fused_experts_fp8_ref(x[rows], q13, w13s.cpu(), q2, w2s.cpu(), tw.cpu()[rows], ids.cpu()[rows],
                                        mirror_rounding=mode)
    _close(out[rows.to(dev)], refm, rtol=3e-2, atol=0.04 * out.float().abs().max().item())


def test_layer_step_replays_from_a_hip_graph(moe, oracle, dev):
    """Routing, alignment and the expert MLP enqueue no allocation of their own,
    no host sync and no memset, so one call can be recorded into a HIP graph.
    Every replay, with eager work and synchronisations in between, must give
    the eager result bit for bit (all kernels are deterministic)."""
    x, w13, w2, logits = _layer(16, 256, 128, 96, 4, 23, torch.bfloat16)
    x, w13, w2, logits = x.to(dev), w13.to(dev), w2.to(dev), logits.to(dev)

    def step(inp):
        tw, ids, _ = moe.fused_topk(inp, logits, 4, True)
        return moe.fused_experts(inp, w13, w2, None, None, tw, ids)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    static_x = x.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = step(static_x)
    for r in range(4):
        fresh = (x * (1.0 + 0.25 * r)).to(torch.bfloat16)
        want = step(fresh).clone()          # eager work between replays
        torch.cuda.synchronize()
        static_x.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out, want), f"replay {r} differs from the eager result"


def _random_cases(n, seed):
    import random
    rnd = random.Random(seed)
    cases = []
    for i in range(n):
        E = rnd.choice([1, 3, 8, 16, 40, 128])
        K = rnd.choice([k for k in (1, 2, 4, 8) if k <= E])
        H = 64 * rnd.randint(1, 8) if rnd.random() < 0.8 else 8 * rnd.randint(3, 40)
        I = 64 * rnd.randint(1, 6) if rnd.random() < 0.7 else 8 * rnd.randint(2, 30)
        T = rnd.choice([1, 2, 7, 33, 64, 100, 257, 700, 1500])
        bm = rnd.choice([0, 0, 32, 64, 128, 256])
        dtype = rnd.choice(["bf16", "bf16", "f16", "fp8"])
        if dtype == "fp8":  # one-byte elements: rows are addressed in 16-byte chunks
            H, I = max(16, H // 16 * 16), max(16, I // 16 * 16)
        cases.append((i, E, K, H, I, T, bm, dtype))
    return cases


# MOE_FUZZ_N / MOE_FUZZ_SEED widen the sweep for a one-off run
@pytest.mark.parametrize("case", _random_cases(int(os.environ.get("MOE_FUZZ_N", "36")),
                                               int(os.environ.get("MOE_FUZZ_SEED", "20250"))),
                         ids=lambda c: "-".join(map(str, c)))
def test_random_shapes_all_kernels(moe, oracle, dev, case, monkeypatch):
    """Seeded random layer shapes, token counts, block sizes and dtypes: every
    dispatch branch (large-tile, streaming, register-staged; 16-bit and e4m3)
    with ragged N / K, empty experts and single tokens, against the oracle that
    rounds where the kernels store."""
    i, E, K, H, I, T, bm, dt = case
    dtype = torch.float16 if dt == "f16" else torch.bfloat16
    x, w13, w2, logits = _layer(E, H, I, T, K, 1000 + i, dtype)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    if bm:
        monkeypatch.setattr(moe.fused_moe, "try_get_optimal_moe_config",
                            lambda *a, **k: {"BLOCK_SIZE_M": bm})
    d = lambda t: t.to(dev)
    if dt == "fp8":
        w13q, w13s, w2q, w2s = moe.quantize_expert_weights(d(w13), d(w2))
        out = moe.fused_experts(d(x), w13q, w2q, None, None, d(tw), d(ids), per_channel_quant=True,
                                w1_scale=w13s, w2_scale=w2s)
        # one e4m3 step of an intermediate element (its 16-bit value landing on the other side of a
        # tie) moves that term by 6 %: the bound stays inside the 6e-2 the fp8 path is held to
        _close_mirrored(out, lambda m: oracle.fused_experts_fp8_ref(
            x, w13q.view(torch.uint8).cpu(), w13s.cpu(), w2q.view(torch.uint8).cpu(), w2s.cpu(), tw, ids,
            mirror_rounding=m), _mode(moe, T, E, K, H, dtype, fp8=True, bm=bm or None), rtol=3e-2,
            atol=0.04 * out.float().abs().max().item() + 1e-6)
    else:
        out = moe.fused_experts(d(x), d(w13), d(w2), None, None, d(tw), d(ids))
        _close_mirrored(out, lambda m: oracle.fused_experts_ref(x, w13, w2, tw, ids, mirror_rounding=m),
                        _mode(moe, T, E, K, H, dtype, bm=bm or None), rtol=1.6e-2,
                        atol=2e-3 + 4e-3 * out.float().abs().max().item())


@pytest.mark.gpu
def test_gpt_oss_mlp_block(moe, oracle, dev):
    """nanovllm/models/gpt_oss.py:120-158: router linear with bias, experts with biases and
    the interleaved swigluoai activation, renormalised top-k.  The routing is checked
    bit-exactly on the router logits the GPU produced, the output against the fp32 oracle."""
    E, H, I, T, K = 32, 256, 128, 90, 4
    g = torch.Generator().manual_seed(17)
    blk = moe.GptOssMLP(E, K, H, I).to(dev)
    ex = blk.experts
    assert ex.activation == "swigluoai" and ex.renormalize and hasattr(ex, "w13_bias")
    blk.router.weight.data.copy_((torch.randn(E, H, generator=g) * 0.05).bfloat16())
    blk.router.bias.data.copy_((torch.randn(E, generator=g) * 0.5).bfloat16())
    ex.w13_weight.data.copy_((torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16())
    ex.w2_weight.data.copy_((torch.randn(E, H, I, generator=g) * 0.05).bfloat16())
    ex.w13_bias.data.copy_((torch.randn(E, 2 * I, generator=g) * 0.1).bfloat16())
    ex.w2_bias.data.copy_((torch.randn(E, H, generator=g) * 0.1).bfloat16())
    x = torch.randn(T, H, generator=g).bfloat16()
    xd = x.to(dev)
    logits = blk.router(xd)
    # the router is a linear in the activation dtype: fp32 sum + bias, one rounding
    want_logits = torch.nn.functional.linear(x.double(), blk.router.weight.data.cpu().double(),
                                             blk.router.bias.data.cpu().double())
    assert ((logits.cpu().double() - want_logits).abs() <= 2.0 ** -7 * want_logits.abs() + 1e-6).all()
    out = blk(xd.clone())
    tw, ids, _ = oracle.topk_softmax(logits.float().cpu(), K, renormalize=True)
    ref = oracle.fused_experts_ref(x, ex.w13_weight.data.cpu(), ex.w2_weight.data.cpu(), tw, ids,
                                   activation="swigluoai", w1_bias=ex.w13_bias.data.cpu(),
                                   w2_bias=ex.w2_bias.data.cpu(), mirror_rounding=True)
    _close(out, ref)
    # and the north-star bound against the oracle that rounds nowhere
    _close(out, oracle.fused_experts_ref(x, ex.w13_weight.data.cpu(), ex.w2_weight.data.cpu(), tw, ids,
                                         activation="swigluoai", w1_bias=ex.w13_bias.data.cpu(),
                                         w2_bias=ex.w2_bias.data.cpu()))


@pytest.mark.gpu
@pytest.mark.parametrize("pattern", ["one_expert", "one_row_each", "two_heavy_rest_single"])
def test_large_tile_ranges_on_lopsided_routing(moe, oracle, dev, pattern, monkeypatch):
    """Alignment blocks of 256 with routings that make the per-XCD work ranges degenerate: every
    block of one expert (ranges cut inside it), one row per expert (weight-streaming blocks
    only), two heavy experts among many single-row ones (ranges of very unequal length)."""
    E, H, I, K = 64, 256, 128, 1
    g = torch.Generator().manual_seed(31)
    if pattern == "one_expert":
        T = 3000
        ids = torch.full((T, 1), 5, dtype=torch.int32)
    elif pattern == "one_row_each":
        T = E
        ids = torch.randperm(E, generator=g).to(torch.int32).view(T, 1)
    else:
        T = 2 * 1500 + (E - 2)
        ids = torch.cat([torch.full((1500,), 7), torch.full((1500,), 40),
                         torch.tensor([e for e in range(E) if e not in (7, 40)])]).to(torch.int32)
        ids = ids[torch.randperm(T, generator=g)].view(T, 1)
    x = torch.randn(T, H, generator=g).bfloat16()
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16()
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).bfloat16()
    tw = torch.rand(T, K, generator=g) + 0.5
    monkeypatch.setattr(moe.fused_moe, "try_get_optimal_moe_config", lambda *a, **k: {"BLOCK_SIZE_M": 256})
    d = lambda t: t.to(dev)
    out = moe.fused_experts(d(x), d(w13), d(w2), None, None, d(tw), d(ids))
    _close_mirrored(out, lambda m: oracle.fused_experts_ref(x, w13, w2, tw, ids, mirror_rounding=m),
                    "fused", rtol=1.6e-2, atol=2e-3 + 4e-3 * out.float().abs().max().item())


@pytest.mark.gpu
@pytest.mark.parametrize("rows_per_expert", [256, 512, 32, 255, 257])
def test_experts_with_exactly_full_blocks(moe, oracle, dev, rows_per_expert):
    """Every expert receives the same number of rows: exact multiples of the 256-slot block
    (no padding slot anywhere: the padded total equals the number of routed rows), of the
    32-slot block, and one row to either side of a block boundary."""
    E, H, I, K = 16, 256, 128, 2
    T = rows_per_expert * E // K
    g = torch.Generator().manual_seed(5 + rows_per_expert)
    t = torch.arange(T).view(T, 1)
    k = torch.arange(K).view(1, K)
    ids = ((t * K + k) * 5 % E).to(torch.int32)            # 5 and E coprime: every expert T K / E rows
    assert torch.bincount(ids.flatten().long(), minlength=E).unique().tolist() == [rows_per_expert]
    x = torch.randn(T, H, generator=g).bfloat16()
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16()
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).bfloat16()
    tw = torch.rand(T, K, generator=g) + 0.5
    d = lambda z: z.to(dev)
    for bm in (256, 32):
        so, eo, npp = moe.fused_moe.moe_align_block_size(d(ids), bm, E)
        oso, oeo, onpp = oracle.moe_align_block_size(ids, bm, E)
        assert torch.equal(so.cpu(), oso) and torch.equal(eo.cpu(), oeo) and int(npp) == int(onpp)
        if rows_per_expert % bm == 0:
            assert int(npp) == T * K
        out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
        moe.fused_moe.launch_fused_experts(d(x), out, d(w13), d(w2), None, None, None, None, d(tw), so, eo, npp, bm)
        mode = _mode(moe, T, E, K, H, torch.bfloat16, bm=bm)
        _close_mirrored(out, lambda m: oracle.fused_experts_ref(x, w13, w2, tw, ids, mirror_rounding=m), mode,
                        rtol=1.6e-2, atol=2e-3 + 4e-3 * out.float().abs().max().item())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("E,H,I,T,K,act", [(16, 512, 256, 2500, 4, "silu"), (8, 256, 192, 3000, 2, "swigluoai"),
                                          (64, 256, 128, 6000, 8, "silu")])
def test_one_launch_form_equals_two_launches(moe, oracle, dev, dtype, E, H, I, T, K, act):
    """Blocks of 256 with 16-bit dtypes enqueue the gate-up and the down pass as one
    launch, the down tiles of an m-block starting once its gate-up tiles are counted
    in.  Same tiles, same arithmetic: the result equals that of two launches bit for
    bit, on every repetition (a down tile that started early would read stale rows)."""
    fm = moe.fused_moe
    x, w13, w2, logits = _layer(E, H, I, T, K, 300 + E, dtype)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    d = lambda t: t.to(dev)
    x, w13, w2, tw, ids = d(x), d(w13), d(w2), d(tw), d(ids)
    so, eo, npp = fm.moe_align_block_size(ids, 256, E)
    two = torch.empty_like(x)
    fm.launch_fused_experts(x, two, w13, w2, None, None, None, None, tw, so, eo, npp, 256, activation=act,
                            passes=7 | 8)
    _close(two, oracle.fused_experts_ref(x.cpu(), w13.cpu(), w2.cpu(), tw.cpu(), ids.cpu(), activation=act))
    ws = None
    for rep in range(6):
        one = torch.full_like(x, float("nan"))
        # a fresh workspace each time: the counters and the intermediate start from whatever memory holds
        fm.launch_fused_experts(x, one, w13, w2, None, None, None, None, tw, so, eo, npp, 256, activation=act)
        torch.cuda.synchronize()
        assert torch.equal(one, two), f"repetition {rep}: {(one != two).sum().item()} elements differ"
    # every hand-off forced across XCDs (passes bit 32: the down tiles of a block run on the XCD next
    # to the one that ran its gate-up tiles, so the intermediate is written through one L2 and read
    # through another): still the same bits
    for rep in range(3):
        far = torch.full_like(x, float("nan"))
        args = fm.launch_fused_experts(x, far, w13, w2, None, None, None, None, tw, so, eo, npp, 256, activation=act,
                                       passes=7 | 32)
        fm.fused_experts_status(args)
        assert torch.equal(far, two), f"cross-XCD repetition {rep}: {(far != two).sum().item()} elements differ"


@pytest.mark.gpu
def test_empty_batch_and_chunk_boundary(moe, oracle, dev):
    """No tokens: empty results, nothing enqueued.  More than 65536 tokens: the
    host loop of nanovllm/layers/for_moe/fused_moe.py:503,547-566 runs the path in
    chunks of 65536 rows, the last one ragged with its own block size."""
    E, H, I, K = 8, 64, 64, 2
    g = torch.Generator().manual_seed(12)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16()
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).bfloat16()
    d = lambda t: t.to(dev)
    x0 = torch.empty(0, H, dtype=torch.bfloat16, device=dev)
    tw0, ids0, tei0 = moe.fused_topk(x0, torch.empty(0, E, device=dev), K, True)
    assert tuple(tw0.shape) == (0, K) and tuple(ids0.shape) == (0, K) and tuple(tei0.shape) == (0, K)
    out0 = moe.fused_experts(x0, d(w13), d(w2), None, None, tw0, ids0)
    assert tuple(out0.shape) == (0, H) and out0.dtype == torch.bfloat16
    T = 65536 + 300
    x = torch.randn(T, H, generator=g).bfloat16()
    logits = torch.randn(T, E, generator=g)
    tw, ids, _ = moe.fused_topk(d(x), d(logits), K, True)
    out = moe.fused_experts(d(x), d(w13), d(w2), None, None, tw, ids)
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, 65536, 4099), torch.arange(65536 - 3, T, 7)])
    ref = oracle.fused_experts_ref(x[rows], w13, w2, tw.cpu()[rows], ids.cpu()[rows])
    _close(out[rows.to(dev)], ref)


@pytest.mark.gpu
def test_one_launch_form_on_two_streams(moe, oracle, dev):
    """Two layers enqueued side by side on two streams, each with its own workspace:
    the one-launch kernels of both share the CUs, and a down tile only ever waits for
    gate-up tiles of its own launch that were started before it.  Results equal the
    ones computed alone, bit for bit."""
    fm = moe.fused_moe
    d = lambda t: t.to(dev)
    jobs = []
    for E, H, I, T, K, seed in ((16, 512, 256, 2500, 4, 71), (64, 256, 128, 6000, 8, 72)):
        x, w13, w2, logits = _layer(E, H, I, T, K, seed, torch.bfloat16)
        tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
        x, w13, w2, tw, ids = d(x), d(w13), d(w2), d(tw), d(ids)
        so, eo, npp = fm.moe_align_block_size(ids, 256, E)
        ws = torch.empty(moe._lib.lib().moe_fused_experts_workspace_bytes(
            T, H, I, E, K, 256, moe._lib.DTYPE_CODE[torch.bfloat16], moe._lib.DTYPE_CODE[torch.bfloat16]),
            dtype=torch.uint8, device=dev)
        alone = torch.empty_like(x)
        fm.launch_fused_experts(x, alone, w13, w2, None, None, None, None, tw, so, eo, npp, 256, workspace=ws)
        jobs.append(dict(x=x, w13=w13, w2=w2, tw=tw, so=so, eo=eo, npp=npp, ws=ws, alone=alone,
                         out=torch.empty_like(x), stream=torch.cuda.Stream(device=dev)))
    torch.cuda.synchronize()
    for rep in range(8):
        for j in jobs:
            with torch.cuda.stream(j["stream"]):
                fm.launch_fused_experts(j["x"], j["out"], j["w13"], j["w2"], None, None, None, None, j["tw"],
                                        j["so"], j["eo"], j["npp"], 256, workspace=j["ws"])
    torch.cuda.synchronize()
    for j in jobs:
        assert torch.equal(j["out"], j["alone"])


@pytest.mark.gpu
def test_expired_wait_of_the_one_launch_form_is_reported(moe, oracle, dev):
    """The down tiles of the one-launch form wait, boundedly, for their block's gate-up
    tiles.  With the wait limit forced to 0 from the host every down tile that finds its
    block incomplete gives up at once (here: all 24 tiles of an XCD start together, so the
    down tiles do meet unfinished blocks).  Such a tile must not multiply a partly written
    intermediate: it writes NaN rows, the status call reports it, every kernel exits
    normally, and the next call with the default limit is clean again."""
    fm = moe.fused_moe
    E, H, I, T, K = 16, 512, 256, 2500, 4
    x, w13, w2, logits = _layer(E, H, I, T, K, 300 + E, torch.bfloat16)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    d = lambda t: t.to(dev)
    x, w13, w2, tw, ids = d(x), d(w13), d(w2), d(tw), d(ids)
    so, eo, npp = fm.moe_align_block_size(ids, 256, E)
    ws = torch.empty(fm.fused_experts_workspace_bytes(T, H, I, E, K, 256, torch.bfloat16), dtype=torch.uint8, device=dev)
    good = torch.empty_like(x)
    args = fm.launch_fused_experts(x, good, w13, w2, None, None, None, None, tw, so, eo, npp, 256, workspace=ws)
    fm.fused_experts_status(args)                       # default limit: nothing expired
    assert not torch.isnan(good).any()
    old = fm.set_wait_limit(0)
    try:
        bad = torch.empty_like(x)
        args = fm.launch_fused_experts(x, bad, w13, w2, None, None, None, None, tw, so, eo, npp, 256, workspace=ws)
        expired = False
        try:
            fm.fused_experts_status(args)
        except RuntimeError as err:
            assert "gave up waiting" in str(err)
            expired = True
        torch.cuda.synchronize()                         # the launch has drained
        # Whether a down tile meets an unfinished block is a matter of timing (it does wherever an
        # XCD has more CUs than a block has gate-up tiles); what must hold either way: the status
        # reports an expiry exactly when NaN rows exist, and every other element is the good one.
        nan_rows = torch.isnan(bad).any(dim=1)
        assert bool(nan_rows.any()) == expired
        clean = ~torch.isnan(bad)
        assert torch.equal(bad[clean], good[clean])
    finally:
        assert fm.set_wait_limit(old) == 0
    if not expired:
        pytest.skip("no down tile met an unfinished block on this GPU: the forced expiry did not occur")
    again = torch.empty_like(x)
    args = fm.launch_fused_experts(x, again, w13, w2, None, None, None, None, tw, so, eo, npp, 256, workspace=ws)
    fm.fused_experts_status(args)
    assert torch.equal(again, good)
    # two launches (passes bit 8) have no hand-off: the status call has nothing to read
    args = fm.launch_fused_experts(x, again, w13, w2, None, None, None, None, tw, so, eo, npp, 256, workspace=ws,
                                   passes=7 | 8)
    fm.fused_experts_status(args)


@pytest.mark.gpu
def test_longer_sorted_ids_buffer_is_accepted_and_its_surplus_ignored(moe, oracle, dev):
    """A C caller may hand over a sorted_token_ids buffer longer than T*K + E*(block-1): the
    workspace layout must not follow the caller's figure (it once did, and the regions
    overlapped).  Same result as with the exact length."""
    fm = moe.fused_moe
    E, H, I, T, K = 8, 256, 128, 1200, 2
    x, w13, w2, logits = _layer(E, H, I, T, K, 55, torch.bfloat16)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    d = lambda t: t.to(dev)
    x, w13, w2, tw, ids = d(x), d(w13), d(w2), d(tw), d(ids)
    for bs in (256, 32):
        so, eo, npp = fm.moe_align_block_size(ids, bs, E)
        exact = torch.empty_like(x)
        fm.launch_fused_experts(x, exact, w13, w2, None, None, None, None, tw, so, eo, npp, bs)
        longer = torch.cat([so, torch.full((5000,), T * K, dtype=torch.int32, device=dev)])
        out = torch.empty_like(x)
        fm.launch_fused_experts(x, out, w13, w2, None, None, None, None, tw, longer, eo, npp, bs)
        torch.cuda.synchronize()
        assert torch.equal(out, exact)
        _close(out, oracle.fused_experts_ref(x.cpu(), w13.cpu(), w2.cpu(), tw.cpu(), ids.cpu()))


def _tile_reference(w: torch.Tensor, gated: bool, interleaved: bool) -> torch.Tensor:
    """The unit order of ``moe_tile_expert_weights`` written out with index arithmetic on
    the CPU: units [expert][rows / 256][K / 64] of 256 rows x 8 chunks of 8 elements; unit
    row r holds source row (gated: gate row 128 nt + r for r < 128, its up row for r >= 128;
    else row 256 nt + r) and its chunk c sits at position c ^ ((r >> 1) & 7)."""
    E, rows, K = w.shape
    n_tiles, k_tiles = rows // 256, K // 64
    r = torch.arange(256)
    nt = torch.arange(n_tiles).view(-1, 1)
    if gated:
        half, n = r // 128, nt * 128 + (r % 128)
        srow = 2 * n + half if interleaved else half * (rows // 2) + n
    else:
        srow = nt * 256 + r
    pos = torch.arange(8)
    chunk = pos.view(1, 8) ^ ((r.view(256, 1) >> 1) & 7)                      # [256, 8]
    src = w.view(E, rows, k_tiles, 8, 8)                                       # [E, row, kt, chunk, 8]
    out = torch.empty(E, n_tiles, k_tiles, 256, 8, 8, dtype=w.dtype)
    for t in range(n_tiles):
        rows_t = src[:, srow[t]]                                               # [E, 256, kt, chunk, 8]
        picked = rows_t[:, r.view(256, 1), :, chunk]                           # [256, 8, E, kt, 8]
        out[:, t] = picked.permute(2, 3, 0, 1, 4)
    return out.reshape(E, rows, K)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("gated,interleaved", [(True, False), (True, True), (False, False)])
def test_tile_expert_weights_is_the_documented_unit_order(moe, dev, dtype, gated, interleaved):
    g = torch.Generator().manual_seed(3)
    w = torch.randn(3, 512, 192, generator=g).to(dtype)
    got = moe.ops.tile_expert_weights(w.to(dev), gated, interleaved)
    torch.cuda.synchronize()
    assert got.shape == w.shape and got.dtype == w.dtype
    assert torch.equal(got.cpu().view(torch.int16), _tile_reference(w, gated, interleaved).view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,K", [(40, 2), (700, 4), (3000, 2)])
@pytest.mark.parametrize("activation,bias", [("silu", False), ("swigluoai", True), ("gelu", False)])
def test_tiled_weights_give_bit_identical_results(moe, oracle, dev, dtype, T, K, activation, bias):
    """Streaming kernel (40 tokens: blocks of 32) and large-tile kernel (blocks of 256, one
    launch for both passes) on weights re-ordered by ``tile_expert_weights``: the same bits
    as on the row-major weights, and within tolerance of the fp32 oracle."""
    E, H, I = 8, 512, 256
    print(f"tiled weights {dtype} T={T} K={K} {activation} bias={bias}", flush=True)
    x, w13, w2, logits = _layer(E, H, I, T, K, 31 + T, dtype, wstd=0.02)  # the benchmark's weight scale
    g = torch.Generator().manual_seed(5)
    b13 = (torch.randn(E, 2 * I, generator=g) * 0.1).to(dtype) if bias else None
    b2 = (torch.randn(E, H, generator=g) * 0.1).to(dtype) if bias else None
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    dv = lambda t: None if t is None else t.to(dev)
    w13d, w2d = w13.to(dev), w2.to(dev)
    plain = moe.fused_experts(x.to(dev), w13d, w2d, dv(b13), dv(b2), tw.to(dev), ids.to(dev), activation=activation)
    w13t = moe.ops.tile_expert_weights(w13d, True, activation == "swigluoai")
    w2t = moe.ops.tile_expert_weights(w2d, False)
    tiled = moe.fused_experts(x.to(dev), w13t, w2t, dv(b13), dv(b2), tw.to(dev), ids.to(dev), activation=activation,
                              weight_layout="tiled")
    torch.cuda.synchronize()
    assert torch.equal(plain.view(torch.int16), tiled.view(torch.int16))
    _close(tiled, oracle.fused_experts_ref(x, w13, w2, tw, ids, activation=activation, w1_bias=b13, w2_bias=b2))


def test_tiled_weights_are_rejected_where_no_kernel_reads_them(moe, oracle, dev, monkeypatch):
    x, w13, w2, logits = _layer(8, 512, 256, 300, 2, 2, torch.bfloat16)
    tw, ids, _ = oracle.topk_softmax(logits, 2, renormalize=True)
    w13t = moe.ops.tile_expert_weights(w13.to(dev), True)
    w2t = moe.ops.tile_expert_weights(w2.to(dev), False)
    monkeypatch.setattr(moe.fused_moe, "try_get_optimal_moe_config", lambda *a, **k: {"BLOCK_SIZE_M": 64})
    with pytest.raises(RuntimeError, match="tiled weights"):
        moe.fused_experts(x.to(dev), w13t, w2t, None, None, tw.to(dev), ids.to(dev), weight_layout="tiled")
    with pytest.raises(RuntimeError, match="not tileable"):
        moe.ops.tile_expert_weights(torch.zeros(2, 200, 64, dtype=torch.bfloat16, device=dev), True)


def test_fused_moe_layer_with_tiled_weights(moe, oracle, dev):
    """``FusedMoE(weight_layout="tiled")``: process_weights_after_loading re-orders the loaded
    parameters once; the forward result equals the row-major layer's bit for bit."""
    E, H, I, T, K = 8, 256, 128, 500, 2
    x, w13, w2, logits = _layer(E, H, I, T, K, 77, torch.bfloat16)
    outs = []
    for layout in ("plain", "tiled"):
        layer = moe.FusedMoE(E, K, H, I, params_dtype=torch.bfloat16, weight_layout=layout).to(dev)
        layer.w13_weight.data.copy_(w13)
        layer.w2_weight.data.copy_(w2)
        layer.process_weights_after_loading()
        assert layer.weights_tiled == (layout == "tiled")
        outs.append(layer(x.to(dev).clone(), logits.to(dev)))
    torch.cuda.synchronize()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    _close(outs[1], oracle.fused_experts_ref(x, w13, w2, tw, ids))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("E,H,I,T,K", [(8, 100, 52, 33, 2), (4, 66, 30, 17, 2), (16, 1001, 333, 200, 4),
                                       (3, 7, 5, 9, 1), (8, 130, 70, 300, 2)])
def test_ragged_hidden_and_intermediate_sizes(moe, oracle, dev, dtype, E, H, I, T, K):
    """H and I that are not multiples of 16 bytes: the reference's Triton kernel masks the K tail
    and the N edge (nanovllm/layers/for_moe/fused_moe.py:191-205,218-223); here both GEMM
    passes run on the element-by-element variant of the register-staged kernel, which rounds
    where the reference stores."""
    print(f"ragged {dtype} E={E} H={H} I={I} T={T} K={K}", flush=True)
    x, w13, w2, logits = _layer(E, H, I, T, K, 3 + H + T, dtype, wstd=0.05 if H < 500 else 0.02)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    out = moe.fused_experts(x.to(dev), w13.to(dev), w2.to(dev), None, None, tw.to(dev), ids.to(dev))
    torch.cuda.synchronize()
    assert out.dtype == dtype and out.shape == x.shape
    if dtype == torch.float32:
        _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids), rtol=1e-4, atol=1e-5)
    else:
        _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids))
        _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids, mirror_rounding=True), rtol=1.6e-2, atol=2e-3)


@pytest.mark.parametrize("bm", [32, 64, 128, 256])
def test_ragged_sizes_with_every_block_size_bias_and_activations(moe, oracle, dev, bm, monkeypatch):
    E, H, I, T, K = 8, 100, 52, 150, 2
    x, w13, w2, logits = _layer(E, H, I, T, K, 31, torch.bfloat16)
    g = torch.Generator().manual_seed(4)
    b13 = (torch.randn(E, 2 * I, generator=g) * 0.1).bfloat16()
    b2 = (torch.randn(E, H, generator=g) * 0.1).bfloat16()
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    monkeypatch.setattr(moe.fused_moe, "try_get_optimal_moe_config", lambda *a, **k: {"BLOCK_SIZE_M": bm})
    d = lambda t: t.to(dev)
    for act in ("silu", "swigluoai", "gelu"):
        print(f"ragged bm={bm} {act}", flush=True)
        out = moe.fused_experts(d(x), d(w13), d(w2), d(b13), d(b2), d(tw), d(ids), activation=act)
        _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids, activation=act, w1_bias=b13, w2_bias=b2,
                                             mirror_rounding=True), rtol=2e-2, atol=4e-3)
        _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids, activation=act, w1_bias=b13, w2_bias=b2))


def test_element_aligned_tensors_and_odd_strides_equal_the_aligned_call(moe, dev):
    """The same numbers behind a base address that is only element-aligned, and behind weight rows
    with a stride that is not a multiple of 16 bytes: the element-by-element kernel rounds where
    the tuned kernels of this block size do, so the results are equal bit for bit."""
    E, H, I, T, K = 8, 128, 64, 70, 2
    x, w13, w2, logits = _layer(E, H, I, T, K, 77, torch.bfloat16)
    d = lambda t: t.to(dev)
    tw, ids, _ = moe.fused_topk(d(x), d(logits), K, True)
    cfg = {"BLOCK_SIZE_M": 64}   # the register-staged kernel in both calls
    import unittest.mock as mock
    with mock.patch.object(moe.fused_moe, "try_get_optimal_moe_config", lambda *a, **k: cfg):
        want = moe.fused_experts(d(x), d(w13), d(w2), None, None, tw, ids)
        xs = torch.empty(T * H + 1, dtype=torch.bfloat16, device=dev)[1:].view(T, H)       # base + 2 bytes
        xs.copy_(x)
        w13s = torch.empty(E, 2 * I, H + 3, dtype=torch.bfloat16, device=dev)[:, :, :H]     # row stride H + 3
        w13s.copy_(w13)
        w2s = torch.empty(E * H * I + 1, dtype=torch.bfloat16, device=dev)[1:].view(E, H, I)
        w2s.copy_(w2)
        assert xs.data_ptr() % 16 != 0 and w13s.stride(1) % 8 != 0
        got = moe.fused_experts(xs, w13s, w2s, None, None, tw, ids)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def _random_ragged_cases(n, seed):
    import random
    rnd = random.Random(seed)
    cases = []
    for i in range(n):
        E = rnd.choice([1, 3, 8, 40])
        K = rnd.choice([k for k in (1, 2, 4) if k <= E])
        H, I = rnd.randint(3, 300), rnd.randint(2, 200)
        if rnd.random() < 0.3:
            H = 64 * rnd.randint(1, 4)          # only I ragged: the gate-up pass alone would suit the tuned kernels
        T = rnd.choice([1, 5, 33, 100, 257, 600])
        bm = rnd.choice([0, 32, 64, 128, 256])
        cases.append((i, E, K, H, I, T, bm, rnd.choice(["bf16", "f16", "f32"])))
    return cases


@pytest.mark.parametrize("case", _random_ragged_cases(16, 4711), ids=lambda c: "-".join(map(str, c)))
def test_random_ragged_shapes(moe, oracle, dev, case, monkeypatch):
    """Seeded random hidden / intermediate sizes with no regard for 16-byte chunks, every block size
    and dtype, against the oracle that rounds where the reference stores."""
    i, E, K, H, I, T, bm, dt = case
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dt]
    x, w13, w2, logits = _layer(E, H, I, T, K, 2000 + i, dtype)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    if bm:
        monkeypatch.setattr(moe.fused_moe, "try_get_optimal_moe_config", lambda *a, **k: {"BLOCK_SIZE_M": bm})
    d = lambda t: t.to(dev)
    out = moe.fused_experts(d(x), d(w13), d(w2), None, None, d(tw), d(ids))
    if dtype == torch.float32:
        _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids), rtol=1e-4, atol=1e-5)
    else:
        ragged = H % 8 != 0 or I % 8 != 0
        mode = True if ragged else _mode(moe, T, E, K, H, dtype, bm=bm or None)
        _close(out, oracle.fused_experts_ref(x, w13, w2, tw, ids, mirror_rounding=mode), rtol=1.6e-2,
               atol=2e-3 + 4e-3 * out.float().abs().max().item())
