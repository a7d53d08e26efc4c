"""GPU parity, bit-exact: router softmax/top-k and expert-sorted alignment
through the C ABI (via the Python ops) against the CPU oracle."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run_topk(moe, g, K, renorm, dev):
    T = g.shape[0]
    w = torch.full((T, K), -7.0, dtype=torch.float32, device=dev)
    ids = torch.full((T, K), -7, dtype=torch.int32, device=dev)
    tei = torch.full((T, K), -7, dtype=torch.int32, device=dev)
    moe.ops.topk_softmax(w, ids, tei, g.to(dev), renormalize=renorm)
    torch.cuda.synchronize()
    return w.cpu(), ids.cpu(), tei.cpu()


@pytest.mark.parametrize("E", [1, 2, 4, 8, 16, 32, 64, 128, 256, 3, 48, 100, 384, 1000, 1024,
                               1025, 1500, 2048, 5000, 16384])
@pytest.mark.parametrize("T", [1, 7, 257])
def test_topk_softmax_bit_exact(moe, oracle, dev, E, T):
    print(f"topk_softmax E={E} T={T}", flush=True)
    g = torch.randn(T, E, generator=torch.Generator().manual_seed(E * 1000 + T)) * 2
    for K in sorted({1, min(2, E), min(8, E), E if E <= 16 else min(8, E)}):
        for renorm in (False, True):
            w, ids, tei = _run_topk(moe, g, K, renorm, dev)
            ow, oids, otei = oracle.topk_softmax(g, K, renormalize=renorm)
            assert torch.equal(ids, oids), (E, T, K, renorm)
            assert torch.equal(tei, otei)
            assert torch.equal(w.view(torch.int32), ow.view(torch.int32)), (E, T, K, renorm)


def test_topk_softmax_wide_rows_ties_subnormals_and_limit(moe, oracle, dev):
    """Rows of more than 1024 columns (the reference's fallback takes any E,
    csrc/moe_topk_softmax_kernels.cu:460-469): equal logits pick the lowest
    indices, a spread that reaches subnormal probabilities ranks as the oracle
    does, and the first unsupported width fails with a message."""
    E = 3000
    g = torch.zeros(5, E)
    w, ids, _ = _run_topk(moe, g, 8, False, dev)
    assert torch.equal(ids, torch.arange(8, dtype=torch.int32).repeat(5, 1))
    gen = torch.Generator().manual_seed(77)
    x = -(torch.rand(33, E, generator=gen) * 40 + 80)
    x[torch.arange(33), torch.randint(0, E, (33,), generator=gen)] = 0.0
    for renorm in (False, True):
        w, ids, tei = _run_topk(moe, x, 16, renorm, dev)
        ow, oids, otei = oracle.topk_softmax(x, 16, renormalize=renorm)
        assert torch.equal(ids, oids) and torch.equal(tei, otei)
        assert torch.equal(w.view(torch.int32), ow.view(torch.int32))
    with pytest.raises(RuntimeError, match="num_experts 16385"):
        _run_topk(moe, torch.zeros(2, 16385), 2, False, dev)


def test_topk_softmax_ties_and_bf16_logits(moe, oracle, dev):
    g = torch.zeros(130, 128)
    w, ids, _ = _run_topk(moe, g, 8, False, dev)
    assert torch.equal(ids, torch.arange(8, dtype=torch.int32).repeat(130, 1))
    gq = torch.randn(4096, 128, generator=torch.Generator().manual_seed(3)).bfloat16().float()
    for renorm in (False, True):
        w, ids, tei = _run_topk(moe, gq, 8, renorm, dev)
        ow, oids, otei = oracle.topk_softmax(gq, 8, renormalize=renorm)
        assert torch.equal(ids, oids) and torch.equal(w.view(torch.int32), ow.view(torch.int32))


def test_topk_softmax_extreme_logits(moe, oracle, dev):
    g = torch.randn(64, 128, generator=torch.Generator().manual_seed(8)) * 40
    g[0, :] = -1e4
    g[1, 5] = 1e4
    w, ids, tei = _run_topk(moe, g, 8, True, dev)
    ow, oids, otei = oracle.topk_softmax(g, 8, renormalize=True)
    assert torch.equal(ids, oids) and torch.equal(w.view(torch.int32), ow.view(torch.int32))


@pytest.mark.parametrize("E", [8, 128, 100])
def test_topk_softmax_subnormal_probabilities_keep_their_rank(moe, oracle, dev, E):
    """Logits 87 to 104 below the row maximum: the reference (built without
    flush-to-zero) ranks their subnormal probabilities by value; below that they are
    exactly zero and the lowest index wins.  Ids and weight bits as the oracle."""
    g = torch.Generator().manual_seed(40 + E)
    T = 96
    x = -(torch.rand(T, E, generator=g) * 40 + 80)         # spread 80 .. 120 below the maximum
    x[torch.arange(T), torch.randint(0, E, (T,), generator=g)] = 0.0
    x[0] = torch.tensor([0.0, -95.0, -101.0, -90.0, -130.0, -99.0, -110.0, -120.0]).repeat(E // 8 + 1)[:E]
    K = min(8, E)
    for renorm in (False, True):
        w, ids, tei = _run_topk(moe, x, K, renorm, dev)
        ow, oids, otei, probs = oracle.topk_softmax(x, K, renormalize=renorm, return_probs=True)
        assert torch.equal(ids, oids), renorm
        assert torch.equal(w.view(torch.int32), ow.view(torch.int32)), renorm
    sub = (probs > 0) & (probs < 2.0 ** -126)
    assert sub.sum() > T                                      # the regime is exercised
    assert ((ow > 0) & (ow < 2.0 ** -126)).any() or renorm    # and reaches the selected weights


def test_fused_topk_matches_oracle_at_full_size(moe, oracle, dev):
    shape, x, logits, _, _ = None, None, None, None, None
    wl = moe.workloads
    x, logits = wl.make_inputs(wl.QWEN3_30B_A3B, 8448, 2, torch.bfloat16)
    w, ids, tei = moe.fused_topk(x.to(dev), logits.to(dev), 8, True)
    ow, oids, otei = oracle.fused_topk(x, logits, 8, True)
    assert torch.equal(ids.cpu(), oids) and torch.equal(tei.cpu(), otei)
    assert torch.equal(w.cpu().view(torch.int32), ow.view(torch.int32))
    # bf16 router logits (what the model hands over) are upcast, ties and all
    w2, ids2, _ = moe.fused_topk(x.to(dev), logits.bfloat16().to(dev), 8, True)
    ow2, oids2, _ = oracle.fused_topk(x, logits.bfloat16().float(), 8, True)
    assert torch.equal(ids2.cpu(), oids2) and torch.equal(w2.cpu().view(torch.int32), ow2.view(torch.int32))


def test_topk_softmax_rejects_bad_arguments(moe, dev):
    g = torch.zeros(4, 8, device=dev)
    w = torch.empty(4, 9, device=dev)
    i = torch.empty(4, 9, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="exceeds num_experts"):
        moe.ops.topk_softmax(w, i, i.clone(), g)
    with pytest.raises(RuntimeError, match="Float"):
        moe.ops.topk_softmax(w[:, :2].contiguous(), i[:, :2].contiguous(), i[:, :2].contiguous(), g.half())
    with pytest.raises(RuntimeError, match="no CPU path"):
        moe.ops.topk_softmax(w.cpu(), i.cpu(), i.cpu(), g.cpu())


# ------------------------------------------------------------------ alignment
ALIGN_CASES = [
    (0, 8, 16), (0, 8, 1), (1, 1, 1), (9, 5, 4), (12, 5, 4), (128, 8, 64), (2048, 128, 16), (2048, 128, 32),
    (2048, 128, 64), (2048, 128, 128), (6144, 128, 64), (16384, 128, 32), (16385, 128, 32),
    (67584, 128, 64), (67584, 128, 128), (67584, 128, 16), (524288, 128, 128), (30000, 60, 7),
    (5000, 1000, 16), (70000, 1024, 8), (3000, 600, 32), (40000, 512, 64), (1000, 2, 256),
    (67584, 128, 256), (100000, 96, 256), (16900, 3, 32), (200000, 256, 64),
]


def _skewed_ids(numel, E, seed):
    g = torch.Generator().manual_seed(seed)
    if numel == 0:
        return torch.zeros(0, dtype=torch.int32)
    p = torch.arange(1, E + 1, dtype=torch.float64) ** -1.1
    p = p[torch.randperm(E, generator=g)]
    return torch.multinomial(p, numel, replacement=True, generator=g).to(torch.int32)


@pytest.mark.parametrize("numel,E,bm", ALIGN_CASES)
def test_moe_align_block_size_bit_exact(moe, oracle, dev, numel, E, bm):
    print(f"align numel={numel} E={E} bm={bm}", flush=True)
    ids = _skewed_ids(numel, E, numel + 7 * E + bm)
    s, e, n = moe.moe_align_block_size(ids.to(dev), bm, E)
    torch.cuda.synchronize()
    os_, oe, on = oracle.moe_align_block_size(ids, bm, E)
    assert n.cpu().item() == on.item()
    assert torch.equal(e.cpu(), oe)
    assert torch.equal(s.cpu(), os_)


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.int16, torch.uint8, torch.int8])
def test_moe_align_block_size_id_dtypes_and_out_of_range_ids(moe, oracle, dev, dtype):
    E = 100
    ids = torch.randint(0, 120, (20000,), generator=torch.Generator().manual_seed(4))  # ids >= E dropped
    if dtype != torch.uint8:
        ids[::97] = -3
    else:
        ids = ids.clamp(min=0)
    ids = ids.to(dtype)
    for n_take in (20000, 3000):
        s, e, n = moe.moe_align_block_size(ids[:n_take].to(dev), 32, E)
        os_, oe, on = oracle.moe_align_block_size(ids[:n_take], 32, E)
        assert torch.equal(s.cpu(), os_) and torch.equal(e.cpu(), oe) and n.cpu().item() == on.item()


def test_moe_align_known_answers_from_reference_comments(moe, dev):
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=torch.int32, device=dev)
    s, e, n = moe.moe_align_block_size(ids, 4, 5)
    assert s[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert n.item() == 16 and e[:4].tolist() == [1, 2, 3, 4]
    ids = torch.tensor([0, 1, 2, 1, 2, 3, 0, 3, 4], dtype=torch.int32, device=dev)
    s, e, n = moe.moe_align_block_size(ids, 4, 5)
    assert s[:20].tolist() == [0, 6, 9, 9, 1, 3, 9, 9, 2, 4, 9, 9, 5, 7, 9, 9, 8, 9, 9, 9]
    assert n.item() == 20


def test_alignment_is_deterministic_and_routed_config_matches(moe, oracle, dev):
    wl = moe.workloads
    x, logits = wl.make_inputs(wl.QWEN3_30B_A3B, 8448, 2, torch.bfloat16)
    _, ids, _ = moe.fused_topk(x.to(dev), logits.to(dev), 8, True)
    first = moe.moe_align_block_size(ids, 128, 128)
    for _ in range(3):
        again = moe.moe_align_block_size(ids, 128, 128)
        assert all(torch.equal(a, b) for a, b in zip(first, again))
    want = oracle.moe_align_block_size(ids.cpu(), 128, 128)
    assert all(torch.equal(a.cpu(), b) for a, b in zip(first, want))


def test_ops_level_align_signature(moe, oracle, dev):
    ids = _skewed_ids(700, 16, 1).to(dev)
    P = 700 + 16 * 31
    s = torch.empty(P, dtype=torch.int32, device=dev)
    e = torch.empty((P + 31) // 32, dtype=torch.int32, device=dev)
    n = torch.empty(1, dtype=torch.int32, device=dev)
    moe.ops.moe_align_block_size(ids, 16, 32, s, e, n)
    os_, oe, on = oracle.moe_align_block_size(ids.cpu(), 32, 16)
    assert torch.equal(s.cpu(), os_) and torch.equal(e.cpu(), oe) and n.item() == on.item()
    with pytest.raises(RuntimeError, match="holds"):
        moe.ops.moe_align_block_size(ids, 16, 32, s[:100].contiguous(), e, n)


# ------------------------------------------------------------------ fused router gate
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,K", [(256, 2048, 128, 8), (700, 512, 64, 4), (33, 256, 32, 2),
                                     (1, 256, 128, 8), (8448, 2048, 128, 8)])
def test_gate_topk_softmax_against_oracle(moe, oracle, dev, dtype, T, H, E, K):
    """Gate GEMM + routing in one kernel.  The logits it routes on (returned
    through logits_out) must be the oracle's logits up to one rounding step of
    the activation dtype (the fp32 sum runs in another order), and the routing
    must be bit-exact for those logits."""
    print(f"gate_topk_softmax {dtype} T={T} H={H} E={E} K={K}", flush=True)
    g = torch.Generator().manual_seed(T + H + E)
    x = torch.randn(T, H, generator=g).to(dtype)
    wg = (torch.randn(E, H, generator=g) * 0.05).to(dtype)
    for renorm in (False, True):
        w = torch.full((T, K), -7.0, dtype=torch.float32, device=dev)
        ids = torch.full((T, K), -7, dtype=torch.int32, device=dev)
        tei = torch.full((T, K), -7, dtype=torch.int32, device=dev)
        logits = torch.full((T, E), float("nan"), dtype=torch.float32, device=dev)
        moe.ops.gate_topk_softmax(w, ids, tei, x.to(dev), wg.to(dev), renormalize=renorm,
                                  logits_out=logits)
        torch.cuda.synchronize()
        got = logits.cpu()
        want = oracle.gate_logits(x, wg)
        # one rounding step of the dtype, plus the fp32 summation-order noise of an
        # H-term dot product where the terms cancel to a small logit
        ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        assert ((got - want).abs() <= 2 * ulp * want.abs() + 3e-5).all()
        assert (got != want).float().mean() < 0.05          # a different rounding is the exception
        assert torch.equal(got, got.to(dtype).float())       # values of the activation dtype
        ow, oids, otei = oracle.topk_softmax(got, K, renormalize=renorm)
        assert torch.equal(ids.cpu(), oids) and torch.equal(tei.cpu(), otei)
        assert torch.equal(w.cpu().view(torch.int32), ow.view(torch.int32))


def test_fused_gate_topk_falls_back_and_block_matches_two_step(moe, oracle, dev, monkeypatch):
    g = torch.Generator().manual_seed(11)
    # unsupported expert count: the gate runs as a plain linear, then fused_topk
    x = torch.randn(50, 256, generator=g).bfloat16().to(dev)
    wg = (torch.randn(48, 256, generator=g) * 0.05).bfloat16().to(dev)
    w, ids, _ = moe.fused_gate_topk(x, wg, 4, True)
    w2, ids2, _ = moe.fused_topk(x, torch.nn.functional.linear(x, wg), 4, True)
    assert torch.equal(ids, ids2) and torch.equal(w, w2)
    with pytest.raises(RuntimeError, match="num_experts 48"):
        moe.ops.gate_topk_softmax(w, ids, ids.clone(), x, wg)
    # the block: gate + experts, against the same experts fed with its own routing
    monkeypatch.setattr(moe.fused_moe, "FUSED_GATE_MIN_TOKENS", 1)   # take the fused kernel at this size
    E, H, I, T, K = 32, 256, 128, 200, 4
    blk = moe.SparseMoeBlock(E, K, H, I, params_dtype=torch.bfloat16).to(dev)
    blk.gate_weight.data.copy_((torch.randn(E, H, generator=g) * 0.05).bfloat16())
    blk.experts.w13_weight.data.copy_((torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16())
    blk.experts.w2_weight.data.copy_((torch.randn(E, H, I, generator=g) * 0.05).bfloat16())
    xs = torch.randn(4, 50, H, generator=g).bfloat16().to(dev)   # leading dims are flattened
    out = blk(xs.clone())
    assert out.shape == xs.shape
    flat = xs.view(-1, H)
    tw, tids, _ = moe.fused_gate_topk(flat, blk.gate_weight.data, K, True)
    ref = moe.fused_experts(flat, blk.experts.w13_weight.data, blk.experts.w2_weight.data, None, None,
                            tw, tids)
    assert torch.equal(out.view(-1, H), ref)
    full = oracle.fused_experts_ref(flat.cpu(), blk.experts.w13_weight.data.cpu(),
                                    blk.experts.w2_weight.data.cpu(), tw.cpu(), tids.cpu())
    assert (out.view(-1, H).float().cpu() - full).abs().max() < 1e-2 + 2e-2 * full.abs().max()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,H", [(1, 8), (7, 2048), (300, 2048), (64, 4096), (33, 1000), (5, 8192), (3, 12288)])
def test_add_rms_norm_against_oracle(moe, oracle, dev, dtype, T, H):
    """csrc/layernorm_kernels.cu:77-108 / :10-35: the residual sum is bit-exact (one fp32
    add, one rounding); the normalised output is rounded twice (before and after the
    weight), so against the float64-variance oracle it may differ by two rounding steps of
    the dtype where the fp32 reduction lands on the other side of a tie."""
    g = torch.Generator().manual_seed(T * 131 + H)
    x = torch.randn(T, H, generator=g).to(dtype)
    res = (torch.randn(T, H, generator=g) * 3).to(dtype)
    w = (1.0 + 0.2 * torch.randn(H, generator=g)).to(dtype)
    step = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -21}[dtype]
    want, want_res = oracle.add_rms_norm(x, res, w, 1e-6)
    out = torch.empty(T, H, dtype=dtype, device=dev)
    res_d = res.to(dev)
    moe.ops.add_rms_norm(out, res_d, x.to(dev), w.to(dev), 1e-6)
    assert torch.equal(res_d.cpu(), want_res)
    diff = (out.cpu().double() - want.double()).abs()
    assert (diff <= 2 * step * want.double().abs() + 1e-30).all()
    if dtype != torch.float32:
        assert (diff > 0).double().mean() < 0.02
    # without a residual; strided rows (a column slice of a wider tensor) and in place
    want2, _ = oracle.add_rms_norm(x, None, w, 1e-5)
    wide = torch.zeros(T, H + 16, dtype=dtype, device=dev)
    xin = wide[:, 8:8 + H]
    xin.copy_(x)
    moe.ops.rms_norm(xin, xin, w.to(dev), 1e-5)
    diff2 = (xin.cpu().double() - want2.double()).abs()
    assert (diff2 <= 2 * step * want2.double().abs() + 1e-30).all()
    assert torch.count_nonzero(wide[:, :8]) == 0 and torch.count_nonzero(wide[:, 8 + H:]) == 0


@pytest.mark.gpu
def test_rms_norm_module_mirrors_the_reference_interface(moe, oracle, dev):
    """nanovllm/layers/layernorm.py:7-34: forward(x) -> out; forward(x, residual) ->
    (out, residual) with the residual updated in place."""
    g = torch.Generator().manual_seed(5)
    norm = moe.RMSNorm(512, eps=1e-6).to(dev).to(torch.bfloat16)
    norm.weight.data.copy_((1.0 + 0.1 * torch.randn(512, generator=g)).bfloat16())
    x = torch.randn(40, 512, generator=g).bfloat16()
    res = torch.randn(40, 512, generator=g).bfloat16()
    res_d = res.to(dev)
    out, res_back = norm(x.to(dev), res_d)
    assert res_back is res_d
    want, want_res = oracle.add_rms_norm(x, res, norm.weight.data.cpu(), 1e-6)
    assert torch.equal(res_d.cpu(), want_res)
    assert ((out.cpu().double() - want.double()).abs() <= 2.0 ** -7 * want.double().abs()).all()
    out1 = norm(x.to(dev))
    want1, _ = oracle.add_rms_norm(x, None, norm.weight.data.cpu(), 1e-6)
    assert ((out1.cpu().double() - want1.double()).abs() <= 2.0 ** -7 * want1.double().abs()).all()
    with pytest.raises(RuntimeError, match="hidden_size"):
        moe.ops.rms_norm(torch.empty(2, 4, 8, device=dev), torch.empty(2, 4, 8, device=dev),
                         torch.ones(8, device=dev), 1e-6)


@pytest.mark.parametrize("T,E,K,skew", [(256, 128, 8, True), (8448, 128, 8, True), (3000, 64, 1, False),
                                        (40, 8, 2, False), (5000, 384, 4, True), (70, 128, 8, True)])
def test_planned_alignment_leaves_the_plan_of_the_plan_kernel(moe, oracle, dev, T, E, K, skew):
    """With blocks of 256 the alignment can also leave, in the workspace of the expert call
    that follows, the per-XCD block ranges and cleared counters which that call otherwise
    computes with a launch of its own (from the aligned ids).  Both must be the same plan,
    and the alignment outputs must not change."""
    fm, L = moe.fused_moe, moe._lib.lib()
    H, I, bm = 256, 128, 256
    code = moe._lib.DTYPE_CODE[torch.bfloat16]
    if skew:
        ids = _skewed_ids(T * K, E, 5 * T + E).view(T, K)
    else:
        ids = torch.randint(0, E, (T, K), generator=torch.Generator().manual_seed(T + E)).to(torch.int32)
    ids = ids.to(dev)
    ws = torch.full((L.moe_fused_experts_workspace_bytes(T, H, I, E, K, bm, code, code),), 0x5a,
                    dtype=torch.uint8, device=dev)
    plan = fm._plan_in_workspace(ws, T, H, I, E, K, bm, code, code, ids.numel())
    assert plan is not None
    b_ptr, d_ptr, n_done, cap_mb = plan
    base = ws.data_ptr()
    got = fm._align_block_size(ids, bm, E, plan)
    want = oracle.moe_align_block_size(ids.cpu(), bm, E)
    assert all(torch.equal(a.cpu(), b) for a, b in zip(got, want))
    words = ws.view(torch.int32)
    bounds = words[(b_ptr - base) // 4:(b_ptr - base) // 4 + 9].cpu()
    done = words[(d_ptr - base) // 4:(d_ptr - base) // 4 + n_done].cpu()
    assert int(done.abs().max()) == 0
    # the plan kernel on the same aligned ids, in a second workspace (gate-up pass only)
    ws2 = torch.full_like(ws, 0x5a)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, H, generator=g).bfloat16().to(dev)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16().to(dev)
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).bfloat16().to(dev)
    tw = torch.rand(T, K, generator=g).to(dev)
    fm.launch_fused_experts(x, torch.empty_like(x), w13, w2, None, None, None, None, tw, *got, bm,
                            workspace=ws2, passes=1)
    torch.cuda.synchronize()
    bounds2 = ws2.view(torch.int32)[(b_ptr - base) // 4:(b_ptr - base) // 4 + 9].cpu()
    assert torch.equal(bounds, bounds2), (bounds.tolist(), bounds2.tolist())
    live = int(got[2].item()) // 256
    assert bounds[0] == 0 and bounds[8] == live and bool((bounds[1:] >= bounds[:-1]).all())
    assert int((bounds[1:] - bounds[:-1]).max()) <= cap_mb


@pytest.mark.parametrize("E,K", [(128, 8), (8, 2), (256, 6), (64, 1), (16, 16)])
@pytest.mark.parametrize("T", [1, 7, 20, 32])
@pytest.mark.parametrize("bm,renorm", [(32, True), (256, True), (64, False)])
def test_route_align_one_launch_equals_the_two_ops(moe, oracle, dev, E, K, T, bm, renorm):
    """``ops.route_align_block_size`` against the oracle's routing and alignment, bit for bit,
    and against the two separate ops."""
    print(f"route_align E={E} K={K} T={T} bm={bm}", flush=True)
    g = torch.Generator().manual_seed(1000 * E + T)
    logits = torch.randn(T, E, generator=g)
    if T > 4:
        logits[3] = logits[2]                      # equal rows route alike
        logits[1] = torch.round(logits[1] * 4) / 4  # ties inside a row: lowest index first
    ow, oids, otei = oracle.topk_softmax(logits, K, renormalize=renorm)
    want = oracle.moe_align_block_size(oids, bm, E)
    ld = logits.to(dev)
    tw = torch.empty(T, K, dtype=torch.float32, device=dev)
    ids = torch.empty(T, K, dtype=torch.int32, device=dev)
    tei = torch.empty(T, K, dtype=torch.int32, device=dev)
    cap = T * K + E * (bm - 1)
    sorted_ids = torch.full((cap,), -7, dtype=torch.int32, device=dev)
    expert_ids = torch.full((-(-cap // bm),), -7, dtype=torch.int32, device=dev)
    npp = torch.full((1,), -7, dtype=torch.int32, device=dev)
    assert moe.ops.route_align_supported(T, E, K)
    moe.ops.route_align_block_size(tw, ids, tei, ld, renorm, E, bm, sorted_ids, expert_ids, npp)
    torch.cuda.synchronize()
    assert torch.equal(ids.cpu(), oids) and torch.equal(tei.cpu(), otei)
    assert torch.equal(tw.cpu().view(torch.int32), ow.view(torch.int32))
    for got, exp in zip((sorted_ids, expert_ids, npp), want):
        assert torch.equal(got.cpu(), exp)


def test_route_align_rejects_what_it_does_not_serve(moe, dev):
    assert not moe.ops.route_align_supported(33, 128, 8)     # one workgroup routes 32 rows at most
    assert not moe.ops.route_align_supported(16, 96, 8)      # not a power of two
    assert not moe.ops.route_align_supported(16, 8, 9)       # top-k beyond the experts
    assert moe.ops.route_align_supported(32, 128, 8)


@pytest.mark.parametrize("T", [5, 32, 64, 500])
@pytest.mark.parametrize("layout", ["plain", "tiled"])
@pytest.mark.parametrize("E,K", [(128, 8), (4, 4)])   # (4, 4) at 32 tokens: blocks of 256, the alignment also plans
def test_fused_topk_experts_equals_the_two_calls(moe, dev, T, layout, E, K):
    """``fused_topk_experts`` (routing + alignment in one launch up to 32 tokens, the two
    calls beyond) gives the bits of ``fused_topk`` followed by ``fused_experts``."""
    H, I = 512, 256
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, H, generator=g).bfloat16().to(dev)
    logits = torch.randn(T, E, generator=g).to(dev)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.02).bfloat16().to(dev)
    w2 = (torch.randn(E, H, I, generator=g) * 0.02).bfloat16().to(dev)
    if layout == "tiled":
        w13, w2 = moe.ops.tile_expert_weights(w13, True), moe.ops.tile_expert_weights(w2, False)
    tw, ids, _ = moe.fused_topk(x, logits, K, True)
    two = moe.fused_experts(x, w13, w2, None, None, tw, ids, weight_layout=layout)
    one = moe.fused_topk_experts(x, logits, w13, w2, K, True, weight_layout=layout)
    torch.cuda.synchronize()
    assert torch.equal(one.view(torch.int16), two.view(torch.int16))
    xin = x.clone()
    ret = moe.fused_topk_experts(xin, logits, w13, w2, K, True, inplace=True, weight_layout=layout)
    assert ret is xin and torch.equal(xin.view(torch.int16), two.view(torch.int16))


def test_fused_topk_experts_inside_a_hip_graph(moe, dev):
    """A call made while the stream is captured enqueues the two kernels (routing, alignment)
    instead of the one launch; every replay gives the bits of the eager call, with eager
    work and synchronisations of the program's own between the replays."""
    T, H, I, E, K = 16, 512, 256, 128, 8
    g = torch.Generator().manual_seed(16)
    x = torch.randn(T, H, generator=g).bfloat16().to(dev)
    logits = torch.randn(T, E, generator=g).to(dev)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.02).bfloat16().to(dev)
    w2 = (torch.randn(E, H, I, generator=g) * 0.02).bfloat16().to(dev)
    assert moe.ops.route_align_supported(T, E, K)
    eager = moe.fused_topk_experts(x, logits, w13, w2, K, True)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        moe.fused_topk_experts(x, logits, w13, w2, K, True)   # warm-up on the capture stream
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            captured = moe.fused_topk_experts(x, logits, w13, w2, K, True)
    torch.cuda.synchronize()
    for rep in range(3):
        captured.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured.view(torch.int16), eager.view(torch.int16)), rep
        again = moe.fused_topk_experts(x, logits, w13, w2, K, True)   # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(again.view(torch.int16), eager.view(torch.int16))
