"""Pins the CPU oracle: known answers from the reference's comments, closed
forms, library routines on special cases and brute force on tiny inputs."""
import math

import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st


# ----------------------------------------------------------------- exp
def test_expf_within_2ulp_of_float64(oracle):
    x = torch.cat([torch.linspace(-87, 0, 200001), torch.linspace(0, 88, 100001),
                   torch.tensor([0.0, -0.0, 1e-8, -1e-8, -86.999, 87.999])]).float()
    y = oracle.expf(x).double().numpy()
    ref = np.exp(x.double().numpy())
    ulp = np.spacing(ref.astype(np.float32)).astype(np.float64)
    err = np.abs(y - ref) / ulp
    assert err.max() <= 2.0, err.max()


def test_expf_special_values(oracle):
    x = torch.tensor([0.0, -105.0, -200.0, 89.0, float("inf"), float("-inf"), float("nan")])
    y = oracle.expf(x)
    assert y[0] == 1.0 and y[1] == 0.0 and y[2] == 0.0
    assert math.isinf(y[3]) and math.isinf(y[4]) and y[5] == 0.0 and math.isnan(y[6])


def test_expf_returns_subnormals_like_an_unflushed_expf(oracle):
    """The reference is compiled without flush-to-zero (setup.py:46-47 passes plain
    -O3 to nvcc), so its expf returns subnormal results for inputs between about
    -87.34 and -103.97 and its router orders experts by them.  The oracle's exp
    does the same: within 2 units of the subnormal spacing (2^-149) of float64
    exp, monotone, non-zero down to ln(2^-149), zero below ln(2^-150)."""
    x = torch.linspace(-104.0, -87.0, 170001).float()
    y = oracle.expf(x).double().numpy()
    ref = np.exp(x.double().numpy())
    ulp = np.maximum(np.spacing(ref.astype(np.float32)).astype(np.float64), 2.0 ** -149)
    assert (np.abs(y - ref) / ulp).max() <= 2.0
    assert (np.diff(y) >= 0).all()
    tiny = 2.0 ** -126
    assert ((y > 0) & (y < tiny)).sum() > 100000          # subnormal results exist and are kept
    assert oracle.expf(torch.tensor([-103.0]))[0] == 2.0 ** -149 * round(math.exp(-103.0) / 2.0 ** -149)
    assert oracle.expf(torch.tensor([-103.2]))[0] > 0 and oracle.expf(torch.tensor([-104.0]))[0] == 0


def test_routing_orders_experts_by_subnormal_probabilities(oracle):
    """Logits 87 to 104 below the row maximum have subnormal probabilities: the
    reference (no flush-to-zero) still ranks them by value, and only below that,
    where they are exactly zero, does the lowest index win."""
    row = torch.tensor([[-120.0, -95.0, 0.0, -101.0, -90.0, -130.0, -99.0, -110.0]])
    w, ids, _, probs = oracle.topk_softmax(row, 8, return_probs=True)
    assert ids[0].tolist() == [2, 4, 1, 6, 3, 0, 5, 7]
    p = probs[0].double()
    assert 0 < p[3] < p[6] < p[1] < p[4] < 2.0 ** -126     # subnormal, ordered by value
    assert p[0] == 0 and p[5] == 0 and p[7] == 0          # below 2^-150: ties, lowest index first
    want = torch.softmax(row.double(), -1)[0]
    assert ((p - want).abs() <= 2.0 ** -148).all()
    # a flush-to-zero build would return [2, 4?, ...] with experts 1, 3, 6 tied at zero: ids 0, 1, 3 ...
    flushed = torch.where(p < 2.0 ** -126, torch.zeros_like(p), p)
    assert torch.argsort(flushed, descending=True, stable=True).tolist() != ids[0].tolist()


def test_expf_is_monotone_on_softmax_range(oracle):
    x = torch.linspace(-30, 0, 2_000_001).float()
    y = oracle.expf(x)
    assert bool((y[1:] >= y[:-1]).all())


# ----------------------------------------------------------------- router
def _softmax64(g):
    return torch.softmax(g.double(), -1)


@pytest.mark.parametrize("E,K", [(1, 1), (2, 1), (4, 2), (8, 2), (16, 4), (32, 8), (64, 6),
                                 (128, 8), (256, 8), (3, 2), (48, 4), (100, 8), (384, 8),
                                 (1000, 5), (1025, 8), (5000, 16)])
def test_topk_softmax_against_float64_softmax(oracle, E, K):
    g = torch.randn(37, E, generator=torch.Generator().manual_seed(E * 31 + K))
    w, ids, tei, probs = oracle.topk_softmax(g, K, return_probs=True)
    p64 = _softmax64(g)
    assert torch.allclose(probs.double(), p64, rtol=2e-6, atol=1e-12)
    # each weight is the probability of its expert; ids distinct; weights non-increasing
    assert torch.equal(w, torch.gather(probs, 1, ids.long()))
    assert all(len(set(r.tolist())) == K for r in ids)
    assert bool((w[:, 1:] <= w[:, :-1]).all())
    # ids are the stable descending order of the probabilities
    order = torch.argsort(probs, dim=-1, descending=True, stable=True)[:, :K]
    assert torch.equal(ids.long(), order)
    T = g.shape[0]
    expect_tei = torch.arange(K)[None, :] * T + torch.arange(T)[:, None]
    assert torch.equal(tei.long(), expect_tei)


def test_topk_softmax_ids_follow_logits_when_probabilities_distinct(oracle):
    g = torch.randn(512, 128, generator=torch.Generator().manual_seed(5))
    w, ids, _, probs = oracle.topk_softmax(g, 8, return_probs=True)
    sp = torch.sort(probs, dim=-1, descending=True).values
    distinct = (sp[:, :9][:, 1:] != sp[:, :9][:, :-1]).all(dim=1)
    assert distinct.float().mean() > 0.9
    by_logit = torch.argsort(g, dim=-1, descending=True, stable=True)[:, :8]
    assert torch.equal(ids.long()[distinct], by_logit[distinct])


def test_topk_softmax_ties_take_lowest_index(oracle):
    g = torch.zeros(3, 16)
    w, ids, _ = oracle.topk_softmax(g, 4)
    assert torch.equal(ids, torch.arange(4, dtype=torch.int32).repeat(3, 1))
    assert torch.equal(w, torch.full((3, 4), 1.0 / 16))
    # bf16-quantised logits produce many exact ties
    gq = torch.randn(200, 128, generator=torch.Generator().manual_seed(9)).bfloat16().float()
    gq = (gq * 4).round() / 4
    w, ids, _, probs = oracle.topk_softmax(gq, 8, return_probs=True)
    order = torch.argsort(probs, dim=-1, descending=True, stable=True)[:, :8]
    assert torch.equal(ids.long(), order)
    # a tie that straddles the cut: the lower expert index must be kept
    for r in range(gq.shape[0]):
        kth = probs[r, ids[r, -1].long()]
        tied = torch.nonzero(probs[r] == kth).flatten()
        chosen = [i for i in ids[r].tolist() if probs[r, i] == kth]
        assert chosen == tied[:len(chosen)].tolist()


def test_topk_softmax_k1_is_argmax_and_kE_is_full_sort(oracle):
    g = torch.randn(50, 32, generator=torch.Generator().manual_seed(3))
    _, ids, _ = oracle.topk_softmax(g, 1)
    assert torch.equal(ids.flatten().long(), g.argmax(-1))
    w, ids, _ = oracle.topk_softmax(g, 32)
    assert torch.equal(ids.long(), torch.argsort(g, dim=-1, descending=True, stable=True))
    assert torch.allclose(w.sum(-1), torch.ones(50), atol=1e-6)


def test_topk_softmax_brute_force_tiny(oracle):
    rng = np.random.default_rng(0)
    for E in (2, 3, 4, 5, 8):
        for _ in range(40):
            g = rng.integers(-3, 4, size=(1, E)).astype(np.float32) / 2
            K = int(rng.integers(1, E + 1))
            w, ids, _ = oracle.topk_softmax(torch.from_numpy(g), K)
            ex = [math.exp(float(v) - float(g.max())) for v in g[0]]
            p = [v / sum(ex) for v in ex]
            pool = list(range(E))
            want = []
            for _k in range(K):
                best = max(pool, key=lambda i: (round(p[i], 9), -i))
                want.append(best)
                pool.remove(best)
            assert ids[0].tolist() == want
            assert np.allclose(w[0].numpy(), [p[i] for i in want], rtol=1e-6)


def test_renormalised_weights_equal_softmax_over_selected_logits(oracle):
    # identity used by the reference's unused torch stand-in
    # (nanovllm/layers/for_moe/moe_easy_kernel.py:17-19)
    g = torch.randn(64, 128, generator=torch.Generator().manual_seed(11))
    w, ids, _ = oracle.topk_softmax(g, 8, renormalize=True)
    sel = torch.gather(g, 1, ids.long())
    assert torch.allclose(w.double(), torch.softmax(sel.double(), -1), rtol=1e-5)
    assert torch.allclose(w.sum(-1), torch.ones(64), atol=1e-6)
    w_raw, _, _ = oracle.topk_softmax(g, 8, renormalize=False)
    s = torch.zeros(64)
    for k in range(8):
        s = s + w_raw[:, k]
    assert torch.equal(w, w_raw / s[:, None])


def test_topk_rejects_k_above_e(oracle):
    with pytest.raises(ValueError):
        oracle.topk_softmax(torch.zeros(2, 4), 5)


# ----------------------------------------------------------------- alignment
def test_align_known_answer_python_docstring(oracle):
    # nanovllm/layers/for_moe/fused_moe.py:42-55 (ids reach 4, so five experts)
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=torch.int32)
    s, e, n = oracle.moe_align_block_size(ids, 4, 5)
    assert s[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert n.item() == 16 and e[:4].tolist() == [1, 2, 3, 4]
    assert set(s[16:].tolist()) == {12} and set(e[4:].tolist()) <= {0}


def test_align_known_answer_cuda_comment(oracle):
    # csrc/moe_align_block_size_kernels.cu:92-95
    ids = torch.tensor([0, 1, 2, 1, 2, 3, 0, 3, 4], dtype=torch.int32)
    s, e, n = oracle.moe_align_block_size(ids, 4, 5)
    P = 9
    assert s[:20].tolist() == [0, 6, P, P, 1, 3, P, P, 2, 4, P, P, 5, 7, P, P, 8, P, P, P]
    assert n.item() == 20 and e[:5].tolist() == [0, 1, 2, 3, 4]


def _align_numpy(ids, bm, E):
    ids = np.asarray(ids).reshape(-1)
    numel = ids.size
    valid = (ids >= 0) & (ids < E)
    order = np.argsort(np.where(valid, ids, E), kind="stable")
    order = order[: valid.sum()]
    cnt = np.bincount(ids[valid], minlength=E)
    pad = (cnt + bm - 1) // bm * bm
    cum = np.concatenate([[0], np.cumsum(pad)])
    P = numel + E * (bm - 1)
    out = np.full(P, numel, dtype=np.int32)
    off = 0
    for e in range(E):
        out[cum[e]:cum[e] + cnt[e]] = order[off:off + cnt[e]]
        off += cnt[e]
    B = (P + bm - 1) // bm
    eid = np.zeros(B, dtype=np.int32)
    for e in range(E):
        eid[cum[e] // bm: cum[e + 1] // bm] = e
    return out, eid, int(cum[-1])


@pytest.mark.parametrize("numel,E,bm", [(0, 4, 4), (1, 1, 1), (9, 5, 4), (128, 8, 64),
                                        (2048, 128, 16), (2048, 128, 64), (5000, 60, 32),
                                        (67584, 128, 128), (3000, 1000, 16)])
def test_align_equals_numpy_stable_argsort(oracle, numel, E, bm):
    rng = np.random.default_rng(numel + E)
    ids = rng.integers(0, E, size=numel).astype(np.int32)
    s, e, n = oracle.moe_align_block_size(torch.from_numpy(ids), bm, E)
    ws, we, wn = _align_numpy(ids, bm, E)
    assert n.item() == wn
    assert np.array_equal(s.numpy(), ws) and np.array_equal(e.numpy(), we)


@settings(max_examples=150, deadline=None)
@given(st.integers(1, 6), st.integers(1, 5), st.lists(st.integers(-1, 7), max_size=40))
def test_align_invariants_brute_force(E, bm, raw):
    import importlib
    oracle = importlib.import_module("oracle.moe_oracle")
    ids = torch.tensor(raw, dtype=torch.int64)
    numel = len(raw)
    s, e, n = oracle.moe_align_block_size(ids, bm, E)
    s, e, n = s.tolist(), e.tolist(), n.item()
    cnt = [sum(1 for v in raw if v == x) for x in range(E)]
    assert n == sum((c + bm - 1) // bm * bm for c in cnt)
    assert all(v == numel for v in s[n:]) and all(v == 0 for v in e[n // bm:])
    real = [v for v in s[:n] if v != numel]
    assert sorted(real) == [i for i, v in enumerate(raw) if 0 <= v < E]
    for b in range(n // bm):
        blk = s[b * bm:(b + 1) * bm]
        toks = [v for v in blk if v != numel]
        assert all(raw[t] == e[b] for t in toks)
        assert toks == sorted(toks)
        assert blk[:len(toks)] == toks  # real ids first, then padding
    pos = {v: i for i, v in enumerate(s[:n]) if v != numel}
    for x in range(E):
        mine = [i for i, v in enumerate(raw) if v == x]
        assert [pos[i] for i in mine] == sorted(pos[i] for i in mine)


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8])
def test_align_id_dtypes_agree(oracle, dtype):
    ids = torch.randint(0, 100, (777,), generator=torch.Generator().manual_seed(1))
    a = oracle.moe_align_block_size(ids.to(torch.int32), 16, 100)
    b = oracle.moe_align_block_size(ids.to(dtype), 16, 100)
    assert all(torch.equal(x, y) for x, y in zip(a, b))


# ----------------------------------------------------------------- activations
def test_silu_and_mul_matches_formula(oracle):
    x = torch.randn(33, 2 * 96, generator=torch.Generator().manual_seed(2)) * 3
    out = oracle.silu_and_mul(x)
    ref = torch.nn.functional.silu(x[:, :96].double()) * x[:, 96:].double()
    assert torch.allclose(out.double(), ref, rtol=3e-6, atol=1e-7)
    xb = x.bfloat16()
    outb = oracle.silu_and_mul(xb)
    refb = (torch.nn.functional.silu(xb[:, :96].float()).bfloat16() * xb[:, 96:])
    diff = (outb.float() - refb.float()).abs()
    assert (diff > 0).float().mean() < 0.01  # only exp's last ulp may flip a bf16 rounding
    assert torch.allclose(outb.float(), refb.float(), rtol=2 ** -7, atol=1e-30)
    xh = x.half()
    outh = oracle.silu_and_mul(xh)
    refh = (torch.nn.functional.silu(xh[:, :96].float()).half() * xh[:, 96:])
    assert torch.allclose(outh.float(), refh.float(), rtol=2 ** -10, atol=1e-7)


def test_swigluoai_matches_formula(oracle):
    x = torch.randn(17, 2 * 64, generator=torch.Generator().manual_seed(4)) * 5
    out = oracle.swigluoai_and_mul(x, 1.702, 7.0)
    g = x[:, 0::2].double().clamp(max=7.0)
    u = x[:, 1::2].double().clamp(-7.0, 7.0)
    ref = (u + 1) * g * torch.sigmoid(1.702 * g)
    assert torch.allclose(out.double(), ref, rtol=3e-6, atol=1e-6)


def _ulp_steps(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance of two 16-bit tensors in representable values (same sign assumed where they differ)."""
    ia, ib = a.view(torch.int16).int(), b.view(torch.int16).int()
    return (ia - ib).abs()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_swigluoai_16bit_is_the_float64_formula_rounded_once(oracle, dtype):
    """The bf16 branch (C) and the fp16 branch (Python) of ``swigluoai_and_mul`` have their own
    interleave indexing: gate = even column, up = odd column, both clamps, one rounding at the
    end.  Against the closed form in float64 rounded once; swapping even and odd, dropping a
    clamp or rounding an intermediate fails it."""
    x = (torch.randn(29, 2 * 48, generator=torch.Generator().manual_seed(8)) * 5).to(dtype)
    out = oracle.swigluoai_and_mul(x, 1.702, 7.0)
    assert out.dtype == dtype and tuple(out.shape) == (29, 48)
    g = x[:, 0::2].double().clamp(max=7.0)
    u = x[:, 1::2].double().clamp(-7.0, 7.0)
    ref = ((u + 1) * g * torch.sigmoid(1.702 * g)).to(dtype)
    steps = _ulp_steps(out, ref)
    assert int(steps.max()) <= 1                    # fp32 evaluation against float64: a rounding tie at most
    assert (steps > 0).float().mean() < 0.01
    assert (x[:, 0::2].float() > 7).any() and (x[:, 1::2].float().abs() > 7).any()   # the clamps were exercised
    swapped = ((g + 1) * u.clamp(max=7.0) * torch.sigmoid(1.702 * u)).to(dtype)       # even/odd exchanged
    assert int(_ulp_steps(out, swapped).max()) > 1


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gelu_and_mul_16bit_rounds_the_activation_then_the_product(oracle, dtype):
    """nanovllm/layers/for_moe/moe_easy_kernel.py:89-98 in a 16-bit dtype: erf GELU of the first
    half rounded to the dtype, times the second half, rounded again."""
    x = (torch.randn(31, 2 * 40, generator=torch.Generator().manual_seed(9)) * 3).to(dtype)
    out = oracle.gelu_and_mul(x)
    g, u = x[:, :40].double(), x[:, 40:].double()
    act = (0.5 * g * (1 + torch.erf(g / 2 ** 0.5))).to(dtype)
    ref = (act.double() * u).to(dtype)
    # (far in the negative tail 1 + erf cancels in fp32: there the values are below 1e-5 and only
    # their absolute distance says anything)
    steps = _ulp_steps(out, ref)
    tail = (out.double() - ref.double()).abs() < 1e-5
    assert bool(((steps <= 1) | tail).all()) and ((steps > 0) & ~tail).float().mean() < 0.01
    halves_swapped = ((0.5 * u * (1 + torch.erf(u / 2 ** 0.5))).to(dtype).double() * g).to(dtype)
    assert int(_ulp_steps(out, halves_swapped).max()) > 1
    once = (0.5 * g * (1 + torch.erf(g / 2 ** 0.5)) * u).to(dtype)                    # a single rounding differs somewhere
    assert not torch.equal(out, once)


# ----------------------------------------------------------------- fp8 helpers
def test_e4m3_quantiser_matches_torch_cast_and_saturates(oracle):
    x = torch.cat([torch.linspace(-448, 448, 100001), torch.tensor([0.0, 1e-4, 2 ** -9, 2 ** -10,
                   0.0009765625 * 1.5, 447.9, 500.0, -1e9])]).float()
    q = oracle.quant_e4m3(x)
    d = oracle.dequant_e4m3(q)
    inr = x.abs() <= 448
    want = x[inr].to(torch.float8_e4m3fn).float()
    assert torch.equal(d[inr], want)
    assert d[-2] == 448.0 and d[-1] == -448.0
    # round trip of every finite code
    codes = torch.tensor([c for c in range(256) if (c & 0x7f) != 0x7f], dtype=torch.uint8)
    vals = oracle.dequant_e4m3(codes)
    again = oracle.dequant_e4m3(oracle.quant_e4m3(vals))
    assert torch.equal(vals, again)


def test_per_channel_and_per_token_scales(oracle):
    w = torch.randn(3, 5, 64, generator=torch.Generator().manual_seed(6)) * 0.02
    q, s = oracle.quant_weight_per_channel(w)
    assert torch.allclose(s, w.abs().amax(-1) / 448)
    deq = oracle.dequant_e4m3(q) * s[..., None]
    assert ((deq - w).abs() <= w.abs().amax(-1, keepdim=True) * 2 ** -4 + 1e-9).all()
    # the largest element of every channel lands on the largest code, and the per-token
    # quantiser is the same function of a row
    assert (oracle.dequant_e4m3(q).abs().amax(-1) == 448).all()
    q0, s0 = oracle.quant_act_per_token(w[0])
    assert torch.equal(q0, q[0]) and torch.equal(s0, s[0])
    # codes are those of the fp32 product with the rounded reciprocal of the scale
    want = oracle.quant_e4m3(w[1] * (torch.tensor(1.0) / s[1])[:, None])
    assert torch.equal(q[1], want)


# ----------------------------------------------------------------- expert MLP
def _rand_layer(E=4, H=64, I=32, T=24, K=2, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(dtype)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.1).to(dtype)
    w2 = (torch.randn(E, H, I, generator=g) * 0.1).to(dtype)
    logits = torch.randn(T, E, generator=g)
    return x, w13, w2, logits


def test_fused_experts_k1_unit_weight_is_a_gated_mlp(oracle):
    x, w13, w2, logits = _rand_layer(K=1)
    ids = logits.argmax(-1, keepdim=True).int()
    w = torch.ones(x.shape[0], 1)
    out = oracle.fused_experts_ref(x, w13, w2, w, ids)
    I = w2.shape[2]
    for t in range(x.shape[0]):
        e = ids[t, 0].item()
        h = torch.nn.functional.linear(x[t], w13[e])
        ref = torch.nn.functional.linear(torch.nn.functional.silu(h[:I]) * h[I:], w2[e])
        assert torch.allclose(out[t], ref, rtol=1e-4, atol=1e-5)


def test_fused_experts_single_expert_is_a_dense_mlp(oracle):
    x, w13, w2, _ = _rand_layer(E=1, K=1)
    ids = torch.zeros(x.shape[0], 1, dtype=torch.int32)
    w = torch.full((x.shape[0], 1), 0.5)
    out = oracle.fused_experts_ref(x, w13, w2, w, ids)
    h = x @ w13[0].t()
    I = w2.shape[2]
    ref = 0.5 * ((torch.nn.functional.silu(h[:, :I]) * h[:, I:]) @ w2[0].t())
    assert torch.allclose(out, ref, rtol=1e-4, atol=1e-5)


def test_fused_experts_linear_in_weights_and_permutation_invariant(oracle):
    x, w13, w2, logits = _rand_layer(T=40, K=2)
    w, ids, _ = oracle.topk_softmax(logits, 2, renormalize=True)
    a = oracle.fused_experts_ref(x, w13, w2, w, ids)
    b = oracle.fused_experts_ref(x, w13, w2, 3 * w, ids)
    assert torch.allclose(b, 3 * a, rtol=1e-5, atol=1e-6)
    z = oracle.fused_experts_ref(x, w13, w2, torch.zeros_like(w), ids)
    assert torch.count_nonzero(z) == 0
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(1))
    c = oracle.fused_experts_ref(x[perm], w13, w2, w[perm], ids[perm])
    assert torch.allclose(c, a[perm], rtol=1e-5, atol=1e-6)
    # weight on the input side commutes for K-slot-wise linear second GEMM only when the
    # activation is evaluated on the scaled input: just check it runs and differs
    d = oracle.fused_experts_ref(x, w13, w2, w, ids, apply_router_weight_on_input=True)
    assert d.shape == a.shape and not torch.allclose(d, a)


def test_mirrored_rounding_stays_close_to_fp32(oracle):
    x, w13, w2, logits = _rand_layer(T=32, K=2, dtype=torch.bfloat16)
    w, ids, _ = oracle.topk_softmax(logits, 2, renormalize=True)
    a = oracle.fused_experts_ref(x, w13, w2, w, ids)
    b = oracle.fused_experts_ref(x, w13, w2, w, ids, mirror_rounding=True)
    assert torch.allclose(a, b, rtol=2e-2, atol=1e-2)
    # one rounding of the gated intermediate instead of three: between the two
    c = oracle.fused_experts_ref(x, w13, w2, w, ids, mirror_rounding="fused")
    assert torch.allclose(a, c, rtol=2e-2, atol=1e-2) and not torch.equal(b, c)
    assert (a - c).abs().mean() <= (a - b).abs().mean()
    # with fp32 activations no mode rounds anything
    xf, wf13, wf2 = x.float(), w13.float(), w2.float()
    assert torch.equal(oracle.fused_experts_ref(xf, wf13, wf2, w, ids, mirror_rounding="fused"),
                       oracle.fused_experts_ref(xf, wf13, wf2, w, ids))


def test_gate_logits_are_the_float64_linear_rounded_once(oracle):
    """The router gate is a bias-free linear whose output has the activation
    dtype: against float64 `linear` rounded to that dtype only a double rounding
    can differ (fp32 sum first), and then by one step."""
    g = torch.Generator().manual_seed(3)
    for dtype, ulp in ((torch.bfloat16, 2.0 ** -7), (torch.float16, 2.0 ** -10)):  # spacing / value, at most
        x = torch.randn(64, 512, generator=g).to(dtype)
        w = (torch.randn(128, 512, generator=g) * 0.05).to(dtype)
        got = oracle.gate_logits(x, w)
        want = torch.nn.functional.linear(x.double(), w.double()).to(dtype).float()
        assert got.dtype == torch.float32 and got.shape == (64, 128)
        assert ((got - want).abs() <= ulp * want.abs() + 1e-7).all()
        assert (got != want).float().mean() < 0.01
        tw, ids, _ = oracle.gate_topk_softmax(x, w, 4, renormalize=True)
        tw2, ids2, _ = oracle.topk_softmax(got, 4, renormalize=True)
        assert torch.equal(ids, ids2) and torch.equal(tw, tw2)


def test_add_rms_norm_known_answers(oracle):
    """Pins the norm oracle on rows whose answer is exact: a dropped residual, a
    variance taken over the wrong values or a missing weight each break one."""
    # s = (3, 4): mean square 12.5, r = 1/sqrt(12.5); the residual carries half of the row
    x = torch.tensor([[3.0, 0.0]])
    res = torch.tensor([[0.0, 4.0]])
    w = torch.tensor([2.0, 0.5])
    out, new_res = oracle.add_rms_norm(x, res, w, 0.0)
    assert torch.equal(new_res, torch.tensor([[3.0, 4.0]]))
    r = 1.0 / (12.5 ** 0.5)
    assert torch.allclose(out, torch.tensor([[3.0 * r * 2.0, 4.0 * r * 0.5]]), rtol=1e-6, atol=0)
    # constant rows: x / |x| * w, exactly, for any power-of-two magnitude
    for c in (0.5, -2.0, 8.0):
        out, _ = oracle.add_rms_norm(torch.full((3, 16), c), None, torch.arange(16.0), 0.0)
        assert torch.equal(out, torch.arange(16.0).expand(3, 16) * (1.0 if c > 0 else -1.0))
    # eps enters under the root: zero rows give zero, tiny rows are damped
    out, _ = oracle.add_rms_norm(torch.zeros(2, 8), None, torch.ones(8), 1e-6)
    assert torch.equal(out, torch.zeros(2, 8))
    out, _ = oracle.add_rms_norm(torch.full((1, 4), 1e-3), None, torch.ones(4), 1e-6)
    assert torch.allclose(out, torch.full((1, 4), 1e-3 / (2e-6 ** 0.5)), rtol=1e-6)
    # 16-bit dtypes: the sum is rounded into the residual, the variance is not
    xb = torch.tensor([[1.0, 2.0 ** -8]], dtype=torch.bfloat16)
    rb = torch.tensor([[2.0 ** -8, 1.0]], dtype=torch.bfloat16)
    out, new_res = oracle.add_rms_norm(xb, rb, torch.ones(2, dtype=torch.bfloat16), 0.0)
    assert torch.equal(new_res, torch.ones(1, 2, dtype=torch.bfloat16))     # 1 + 2^-8 rounds (to even) to 1 in bf16
    assert torch.equal(out, torch.full((1, 2), 1.0 - 2.0 ** -8).to(torch.bfloat16))  # r = 1/(1 + 2^-8), not 1
    # against the float64 textbook formula on random rows, one rounding step at most
    g = torch.Generator().manual_seed(11)
    x = torch.randn(32, 256, generator=g).bfloat16()
    res = torch.randn(32, 256, generator=g).bfloat16()
    w = (1.0 + 0.1 * torch.randn(256, generator=g)).bfloat16()
    out, new_res = oracle.add_rms_norm(x, res, w, 1e-6)
    s64 = x.double() + res.double()
    assert torch.equal(new_res, s64.to(torch.bfloat16))
    want = new_res.double() / torch.sqrt((s64 * s64).mean(-1, keepdim=True) + 1e-6) * w.double()
    assert ((out.double() - want).abs() <= 2.0 ** -7 * want.abs() + 1e-12).all()


# ----------------------------------------------------------------- expert MLP: every branch
def _mlp64(x, w13, w2, act, b13=None, b2=None, in_weight=None, out_weight=None):
    """One expert's gated MLP written with torch library routines in float64:
    the textbook form the branches of ``fused_experts_ref`` are pinned to
    (nanovllm/layers/for_moe/fused_moe.py:207-214 bias then routed weight;
    csrc/activation_kernels.cu:8-64; moe_easy_kernel.py:89-98)."""
    F = torch.nn.functional
    h = F.linear(x.double(), w13.double(), None if b13 is None else b13.double())
    if in_weight is not None:
        h = h * in_weight.double()[:, None]           # weight multiplies sum + bias
    I = w2.shape[-1]
    if act == "silu":
        a = F.silu(h[:, :I]) * h[:, I:]
    elif act == "gelu":
        a = F.gelu(h[:, :I]) * h[:, I:]                # erf form, gate = first half
    else:                                              # swigluoai: gate/up interleaved, clamped
        g, u = h[:, 0::2].clamp(max=7.0), h[:, 1::2].clamp(-7.0, 7.0)
        a = (u + 1.0) * g * torch.sigmoid(1.702 * g)
    o = F.linear(a, w2.double(), None if b2 is None else b2.double())
    if out_weight is not None:
        o = o * out_weight.double()[:, None]
    return o


@pytest.mark.parametrize("act", ["silu", "gelu", "swigluoai"])
@pytest.mark.parametrize("on_input", [False, True])
@pytest.mark.parametrize("bias", [False, True])
def test_fused_experts_branches_against_library_mlp(oracle, act, on_input, bias):
    """K=1 per token, several experts: each token's row must be the float64 library
    MLP of its expert, with the bias added before the routed weight multiplies and
    the weight applied on the chosen side.  A swapped gate/up half, a bias added
    after the weight, tanh instead of erf GELU, a missing clamp or de-interleave,
    or the weight applied on both / neither side each fail this."""
    E, H, I, T = 3, 48, 40, 29
    g = torch.Generator().manual_seed(100 + len(act) + 2 * on_input + bias)
    x = torch.randn(T, H, generator=g) * 1.5            # large enough for the swigluoai clamps to bite
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.4
    w2 = torch.randn(E, H, I, generator=g) * 0.2
    b13 = torch.randn(E, 2 * I, generator=g) if bias else None
    b2 = torch.randn(E, H, generator=g) if bias else None
    ids = torch.randint(0, E, (T, 1), generator=g).int()
    w = torch.rand(T, 1, generator=g) + 0.25
    out = oracle.fused_experts_ref(x, w13, w2, w, ids, activation=act, w1_bias=b13, w2_bias=b2,
                                   apply_router_weight_on_input=on_input)
    want = torch.zeros(T, H, dtype=torch.float64)
    for e in range(E):
        sel = (ids[:, 0] == e).nonzero().flatten()
        want[sel] = _mlp64(x[sel], w13[e], w2[e], act, None if b13 is None else b13[e],
                           None if b2 is None else b2[e],
                           in_weight=w[sel, 0] if on_input else None,
                           out_weight=None if on_input else w[sel, 0])
    if act == "swigluoai":
        assert (x @ w13[0].t()).abs().max() > 7.0       # the clamp is exercised
    assert torch.allclose(out.double(), want, rtol=2e-5, atol=2e-5)
    # the two sides of the weight differ (the activation is not linear), so the flag matters
    other = oracle.fused_experts_ref(x, w13, w2, w, ids, activation=act, w1_bias=b13, w2_bias=b2,
                                     apply_router_weight_on_input=not on_input)
    assert not torch.allclose(out, other, rtol=1e-3, atol=1e-3)


def test_fused_experts_topk_combine_is_the_plain_sum(oracle):
    """K=3: the result is the sum over k of the K=1 results (moe_easy_kernel.py:26-31),
    and a bias on the down projection is counted once per selected expert, scaled by
    that expert's routed weight."""
    E, H, I, T, K = 5, 32, 24, 17, 3
    g = torch.Generator().manual_seed(77)
    x = torch.randn(T, H, generator=g)
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.3
    w2 = torch.randn(E, H, I, generator=g) * 0.3
    b2 = torch.randn(E, H, generator=g)
    logits = torch.randn(T, E, generator=g)
    w, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    out = oracle.fused_experts_ref(x, w13, w2, w, ids, w2_bias=b2)
    parts = sum(oracle.fused_experts_ref(x, w13, w2, w[:, k:k + 1], ids[:, k:k + 1], w2_bias=b2)
                for k in range(K))
    assert torch.allclose(out, parts, rtol=1e-5, atol=1e-6)
    want = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for k in range(K):
            e = ids[t, k].item()
            want[t] += _mlp64(x[t:t + 1], w13[e], w2[e], "silu", b2=b2[e], out_weight=w[t:t + 1, k])[0]
    assert torch.allclose(out.double(), want, rtol=2e-5, atol=2e-5)


def _bf(v):
    return torch.as_tensor(v, dtype=torch.float32).bfloat16().float()


def test_mirror_rounding_step_by_step_on_a_2x2_case(oracle):
    """Every rounding point of the two mirrored modes on a case small enough to
    follow by hand (H = 2, I = 1, E = 1, K = 1): the values are chosen so that each
    rounding changes the bf16 result, hence a missing or extra rounding fails."""
    x = torch.tensor([[1.5390625, -0.29296875]]).bfloat16()
    w13 = torch.tensor([[[-2.171875, 0.5703125], [-1.0859375, -1.3984375]]]).bfloat16()   # gate row, up row
    w2 = torch.tensor([[[0.404296875], [0.83984375]]]).bfloat16()
    tw = torch.tensor([[0.7]])
    ids = torch.zeros(1, 1, dtype=torch.int32)
    xf, w13f, w2f = x.float(), w13.float(), w2.float()
    gate32 = xf[0, 0] * w13f[0, 0, 0] + xf[0, 1] * w13f[0, 0, 1]
    up32 = xf[0, 0] * w13f[0, 1, 0] + xf[0, 1] * w13f[0, 1, 1]
    silu = lambda v: v / (1 + torch.exp(-v))
    # mirror_rounding=True: GEMM1 -> bf16, silu -> bf16, product -> bf16, weighted GEMM2 -> bf16, sum -> bf16
    g16, u16 = _bf(gate32), _bf(up32)
    assert g16 != gate32 and u16 != up32                              # the first rounding bites
    s16 = _bf(oracle.silu_and_mul(torch.stack([g16, torch.tensor(1.0)])[None].bfloat16()).float()[0, 0])
    assert s16 == _bf(silu(g16)) and s16 != silu(g16)
    c2 = _bf(s16 * u16)
    assert c2 != s16 * u16
    want_true = torch.stack([_bf(_bf((c2 * w2f[0, r, 0]) * tw[0, 0])) for r in range(2)])
    got_true = oracle.fused_experts_ref(x, w13, w2, tw, ids, mirror_rounding=True)
    assert torch.equal(got_true[0], want_true)
    # mirror_rounding="fused": silu(gate) * up on the fp32 sums, one rounding
    c2f = _bf(silu(gate32) * up32)
    want_fused = torch.stack([_bf((c2f * w2f[0, r, 0]) * tw[0, 0]) for r in range(2)])
    got_fused = oracle.fused_experts_ref(x, w13, w2, tw, ids, mirror_rounding="fused")
    assert torch.equal(got_fused[0], want_fused)
    assert c2f != c2 and not torch.equal(got_fused, got_true)         # the modes are told apart here
    # and the pure fp32 mode rounds nowhere
    want32 = torch.stack([(silu(gate32) * up32 * w2f[0, r, 0]) * tw[0, 0] for r in range(2)])
    got32 = oracle.fused_experts_ref(x, w13, w2, tw, ids)
    assert torch.allclose(got32[0], want32, rtol=1e-6, atol=0) and not torch.equal(got32, got_fused)


def test_mirror_rounding_step_by_step_gelu_and_swigluoai(oracle):
    """The mirrored mode with the other two activations on the same hand-sized case: GEMM1
    rounded, the activation rounded where the reference's kernels round it (gelu: activation,
    then product; swigluoai: once, gate = row 0 and up = row 1 of the interleaved pair), weighted
    GEMM2 rounded, sum rounded."""
    x = torch.tensor([[1.5390625, -0.29296875]]).bfloat16()
    w13 = torch.tensor([[[-2.171875, 0.5703125], [-1.0859375, -1.3984375]]]).bfloat16()
    w2 = torch.tensor([[[0.404296875], [0.83984375]]]).bfloat16()
    tw = torch.tensor([[0.7]])
    ids = torch.zeros(1, 1, dtype=torch.int32)
    xf, w13f, w2f = x.float(), w13.float(), w2.float()
    r0 = _bf(xf[0, 0] * w13f[0, 0, 0] + xf[0, 1] * w13f[0, 0, 1])    # row 0 of w13 after GEMM1, rounded
    r1 = _bf(xf[0, 0] * w13f[0, 1, 0] + xf[0, 1] * w13f[0, 1, 1])    # row 1
    finish = lambda c2: torch.stack([_bf(_bf((c2 * w2f[0, r, 0]) * tw[0, 0])) for r in range(2)])
    # gelu: halves layout (I = 1: row 0 gate, row 1 up); erf form in float64, rounded, product rounded
    act = _bf(0.5 * r0.double() * (1 + torch.erf(r0.double() / 2 ** 0.5)))
    c2 = _bf(act * r1)
    assert c2 != act * r1 or act != 0.5 * r0 * (1 + torch.erf(r0 / 2 ** 0.5))   # a rounding bites
    got = oracle.fused_experts_ref(x, w13, w2, tw, ids, activation="gelu", mirror_rounding=True)
    assert torch.equal(got[0], finish(c2))
    # swigluoai: interleaved pair (row 0 gate, row 1 up), clamps inactive here, one rounding
    a, lim = 1.702, 7.0
    g64, u64 = r0.double().clamp(max=lim), r1.double().clamp(-lim, lim)
    c2s = _bf((u64 + 1) * g64 * torch.sigmoid(a * g64))
    got = oracle.fused_experts_ref(x, w13, w2, tw, ids, activation="swigluoai", mirror_rounding=True)
    assert torch.equal(got[0], finish(c2s))
    # gate and up exchanged would be another number
    c2x = _bf((g64 + 1) * u64.clamp(max=lim) * torch.sigmoid(a * u64))
    assert not torch.equal(finish(c2x), finish(c2s))


# ----------------------------------------------------------------- fp8 expert MLP
def _fp8_cast(t):
    """torch's own e4m3fn rounding (saturating inputs are never passed)."""
    return t.to(torch.float8_e4m3fn).float()


def _fp8_layer(seed, E=3, H=64, I=32, T=21):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(T, H, generator=g) * torch.logspace(-2, 2, T)[:, None]).bfloat16()   # rows of very different size
    # output channels of very different size: a scale applied along the wrong axis cannot pass
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.2 * (2.0 ** (torch.arange(2 * I) % 7 - 3))[None, :, None]
    w2 = torch.randn(E, H, I, generator=g) * 0.2 * (2.0 ** (torch.arange(H) % 5 - 2))[None, :, None]
    return x, w13, w2, g


def test_fp8_reference_step_by_step_against_library_routines(oracle):
    """K=1: per token, x is quantised per row, multiplied with the dequantised
    per-channel weights, gated, quantised per row *again* and multiplied with the
    dequantised down weights.  Every step here uses torch's e4m3 cast and
    F.linear, with wildly non-uniform row and channel magnitudes, so a scale on
    the wrong axis, a missing second quantisation, a dropped routed weight or a
    static (per-tensor) activation scale each fail."""
    F = torch.nn.functional
    x, w13, w2, g = _fp8_layer(5)
    E, T, I = w13.shape[0], x.shape[0], w2.shape[2]
    q13, s13 = oracle.quant_weight_per_channel(w13)
    q2, s2 = oracle.quant_weight_per_channel(w2)
    assert s13.shape == (E, 2 * I) and s2.shape == (E, w2.shape[1])
    assert s13.max() / s13.min() > 30 and s2.max() / s2.min() > 8
    ids = torch.randint(0, E, (T, 1), generator=g).int()
    tw = torch.rand(T, 1, generator=g) + 0.25
    got = oracle.fused_experts_fp8_ref(x, q13, s13, q2, s2, tw, ids)
    xf = x.float()
    sx = xf.abs().amax(-1) / 448.0
    xd = _fp8_cast(xf * (1.0 / sx)[:, None]) * sx[:, None]
    want = torch.zeros(T, w2.shape[1])
    for t in range(T):
        e = ids[t, 0].item()
        W1 = _fp8_cast(w13[e] * (1.0 / s13[e])[:, None]) * s13[e][:, None]
        W2 = _fp8_cast(w2[e] * (1.0 / s2[e])[:, None]) * s2[e][:, None]
        h = F.linear(xd[t], W1)
        a = F.silu(h[:I]) * h[I:]
        sa = a.abs().amax() / 448.0
        ad = _fp8_cast(a * (1.0 / sa)) * sa
        want[t] = F.linear(ad, W2) * tw[t, 0]
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-6 * want.abs().max().item())
    # without the second quantisation the result is measurably different
    nore = torch.zeros_like(want)
    for t in range(T):
        e = ids[t, 0].item()
        W1 = oracle.dequant_e4m3(q13[e]) * s13[e][:, None]
        W2 = oracle.dequant_e4m3(q2[e]) * s2[e][:, None]
        h = F.linear(xd[t], W1)
        nore[t] = F.linear(F.silu(h[:I]) * h[I:], W2) * tw[t, 0]
    assert not torch.allclose(got, nore, rtol=1e-3, atol=1e-3 * want.abs().max().item())


def test_fp8_reference_equals_the_16bit_reference_up_to_one_requantisation(oracle):
    """Weights and activations that e4m3 holds exactly (code values times a
    power-of-two row scale) pass through both quantisers unchanged, so the fp8
    reference may differ from ``fused_experts_ref`` on the same tensors only by
    the re-quantisation of the gated intermediate: at most half an e4m3 step
    (2^-4 relative; 2^-10 of the row scale in the subnormal range) per element,
    propagated through |W2|."""
    g = torch.Generator().manual_seed(8)
    E, H, I, T, K = 4, 64, 32, 26, 2
    codes = torch.tensor([c for c in range(256) if (c & 0x7f) not in (0x7f,)], dtype=torch.uint8)
    vals = oracle.dequant_e4m3(codes)

    def exact(shape, row_exp):
        pick = vals[torch.randint(0, vals.numel(), shape, generator=g)]
        pick[..., 0] = 448.0                               # every row reaches the largest code
        return pick * (2.0 ** row_exp)[..., None]

    x = exact((T, H), torch.randint(-12, -6, (T,), generator=g).float()).bfloat16()
    w13 = exact((E, 2 * I, H), torch.randint(-14, -9, (E, 2 * I), generator=g).float())
    w2 = exact((E, H, I), torch.randint(-13, -8, (E, H), generator=g).float())
    assert torch.equal(x.float().bfloat16(), x)            # 4-bit mantissas: bf16 holds them
    q13, s13 = oracle.quant_weight_per_channel(w13)
    q2, s2 = oracle.quant_weight_per_channel(w2)
    assert torch.equal(oracle.dequant_e4m3(q13) * s13[..., None], w13)      # lossless
    assert torch.equal(oracle.dequant_e4m3(q2) * s2[..., None], w2)
    xq, xs = oracle.quant_act_per_token(x)
    assert torch.equal(oracle.dequant_e4m3(xq) * xs[:, None], x.float())
    logits = torch.randn(T, E, generator=g)
    tw, ids, _ = oracle.topk_softmax(logits, K, renormalize=True)
    got = oracle.fused_experts_fp8_ref(x, q13, s13, q2, s2, tw, ids)
    ref = oracle.fused_experts_ref(x.float(), w13, w2, tw, ids)
    bound = torch.zeros(T, H)
    for t in range(T):
        for k in range(K):
            e = ids[t, k].item()
            h = w13[e] @ x[t].float()
            a = torch.nn.functional.silu(h[:I]) * h[I:]
            step = torch.maximum(a.abs() * 2.0 ** -4, (a.abs().amax() / 448.0) * 2.0 ** -10)
            bound[t] += tw[t, k] * (w2[e].abs() @ step)
    err = (got - ref).abs()
    assert (err <= bound * 1.001 + 1e-7 * ref.abs().max()).all()
    assert err.max() > 0.05 * bound.max()                  # and the re-quantisation is really there


def test_fp8_mirrored_modes_round_where_the_kernels_store(oracle):
    """mirror_rounding=True / "fused" of the fp8 reference: same steps as the
    library recomputation above with the 16-bit roundings inserted."""
    F = torch.nn.functional
    x, w13, w2, g = _fp8_layer(9, E=2, T=9)
    I = w2.shape[2]
    q13, s13 = oracle.quant_weight_per_channel(w13)
    q2, s2 = oracle.quant_weight_per_channel(w2)
    ids = torch.randint(0, 2, (9, 1), generator=g).int()
    tw = torch.rand(9, 1, generator=g) + 0.25
    xf = x.float()
    sx = xf.abs().amax(-1) / 448.0
    xd = _fp8_cast(xf * (1.0 / sx)[:, None]) * sx[:, None]
    r16 = lambda t: t.bfloat16().float()
    for mode in (True, "fused"):
        got = oracle.fused_experts_fp8_ref(x, q13, s13, q2, s2, tw, ids, mirror_rounding=mode)
        want = torch.zeros_like(got)
        for t in range(9):
            e = ids[t, 0].item()
            W1 = oracle.dequant_e4m3(q13[e]) * s13[e][:, None]
            W2 = oracle.dequant_e4m3(q2[e]) * s2[e][:, None]
            h = F.linear(xd[t], W1)
            if mode is True:
                h = r16(h)
                a = r16(r16(oracle.silu_and_mul(torch.cat([h[:I], torch.ones(I)])[None].bfloat16()).float()[0])
                        * h[I:])
            else:
                a = r16(h[:I] / (1 + torch.exp(-h[:I])) * h[I:])
            sa = a.abs().amax() / 448.0
            ad = _fp8_cast(a * (1.0 / sa)) * sa
            want[t] = r16(r16(F.linear(ad, W2) * tw[t, 0]))
        assert torch.allclose(got, want, rtol=2.0 ** -7, atol=1e-6 * want.abs().max().item()), mode
        assert (got != want).float().mean() < 0.02, mode    # only fp32 summation order can flip a rounding


def test_quantiser_scale_floor_for_near_subnormal_rows(oracle):
    """A row whose largest magnitude is tiny but not zero: amax / 448 would have a
    reciprocal that overflows (zeros would turn into NaN codes, the rest saturate).
    The scale is floored at 2^-100 instead; codes stay finite and the round trip is
    still within half an e4m3 step of that scale."""
    x = torch.zeros(4, 16)
    x[0, 3] = 1e-38                     # 1 / (amax / 448) would be +inf
    x[0, 4] = 1e-40                     # subnormal input
    x[1, 5] = -192 * 2.0 ** -100
    x[1, 6] = 2.0 ** -109               # smallest e4m3 subnormal at the floor scale
    x[2, 1] = 448 * 2.0 ** -100         # exactly at the floor
    q, s = oracle.quant_act_per_token(x)
    assert s.tolist() == [2.0 ** -100, 2.0 ** -100, 2.0 ** -100, 1.0]
    assert not ((q & 0x7f) == 0x7f).any()                     # no NaN code
    assert q[3].count_nonzero() == 0 and q[0].count_nonzero() == 0 and q[2, 1] == 0x7e
    assert q[1, 5] == (0x80 | 0x74) and q[1, 6] == 0x01       # -192 = -1.5 * 2^7; 2^-9
    d = oracle.dequant_e4m3(q) * s[:, None]
    assert ((d - x).abs() <= 2.0 ** -100 * 2.0 ** -10 + x.abs() * 2.0 ** -4).all()
    qw, sw = oracle.quant_weight_per_channel(x[None])
    assert torch.equal(qw[0], q) and torch.equal(sw[0], s)
