"""The entry point that allocates nothing (``moe_align_block_size_static``) against
``moe_align_block_size``, through the C ABI: bit-exact on every output, on two calls
in a row that share the library's built-in scratch array, the second smaller."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _align_both(moe, dev, numel, E, bs, seed, dtype=torch.int32):
    L = moe._lib.lib()
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, E, (numel,), generator=g).to(dtype).to(dev)
    cap = numel + E * (bs - 1)
    nblk = (cap + bs - 1) // bs
    stream = torch.cuda.current_stream(dev).cuda_stream
    code = moe._lib.ID_DTYPE_CODE[dtype]
    outs = []
    for static in (False, True):
        # poisoned outputs: every element must be written by the call
        s = torch.full((cap,), -7, dtype=torch.int32, device=dev)
        e = torch.full((nblk,), -7, dtype=torch.int32, device=dev)
        n = torch.full((1,), -7, dtype=torch.int32, device=dev)
        if static:
            rc = L.moe_align_block_size_static(ids.data_ptr(), code, numel, E, bs, s.data_ptr(), cap,
                                               e.data_ptr(), nblk, n.data_ptr(), stream)
        else:
            ws_bytes = L.moe_align_workspace_bytes(numel, E)
            ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
            rc = L.moe_align_block_size(ids.data_ptr(), code, numel, E, bs, s.data_ptr(), cap, e.data_ptr(),
                                        nblk, n.data_ptr(), ws.data_ptr(), ws_bytes, stream)
        assert rc == 0, L.moe_last_error().decode()
        torch.cuda.synchronize()
        outs.append((s.cpu(), e.cpu(), n.cpu()))
    return ids.cpu(), outs


def test_static_alignment_equals_the_workspace_form_on_consecutive_calls(moe, oracle, dev):
    # both sizes are beyond the single-workgroup path, so both use the scratch array;
    # the second call is smaller and finds the first call's histograms in it
    for numel, E, bs, seed in ((67584, 128, 256, 1), (20000, 60, 32, 2), (40000, 1000, 16, 3), (300, 8, 4, 4)):
        print(f"static alignment numel={numel} E={E} block={bs}", flush=True)
        ids, (plain, static) = _align_both(moe, dev, numel, E, bs, seed)
        for a, b in zip(plain, static):
            assert torch.equal(a, b)
        want = oracle.moe_align_block_size(ids, bs, E)
        for a, b in zip(static, want):
            assert torch.equal(a, b)


def test_static_alignment_rejects_sizes_beyond_its_scratch(moe, dev):
    L = moe._lib.lib()
    numel, E, bs = 600_000, 1024, 16           # 1172 segments x 1024 experts x 4 B > 4 MiB
    assert L.moe_align_workspace_bytes(numel, E) > 4 << 20
    one = torch.zeros(1, dtype=torch.int32, device=dev)
    rc = L.moe_align_block_size_static(one.data_ptr(), 0, numel, E, bs, one.data_ptr(), numel + E * (bs - 1),
                                       one.data_ptr(), (numel + E * (bs - 1) + bs - 1) // bs, one.data_ptr(), None)
    assert rc == -3 and b"built-in buffer" in L.moe_last_error()


def test_static_alignment_wrapper(moe, oracle, dev):
    ids = torch.randint(0, 128, (8448, 8), generator=torch.Generator().manual_seed(5), dtype=torch.int32)
    cap = ids.numel() + 128 * 63
    s = torch.empty(cap, dtype=torch.int32, device=dev)
    e = torch.empty((cap + 63) // 64, dtype=torch.int32, device=dev)
    n = torch.empty(1, dtype=torch.int32, device=dev)
    moe.ops.moe_align_block_size_static(ids.to(dev), 128, 64, s, e, n)
    want = oracle.moe_align_block_size(ids, 64, 128)
    assert torch.equal(s.cpu(), want[0]) and torch.equal(e.cpu(), want[1]) and torch.equal(n.cpu(), want[2])
