"""Routing glue of the expert MLP (device-side sort / gather / combine) against the CPU oracle: the sort is
integer work and must match a stable torch sort exactly; the gather is a copy (bit-exact); the combine and the
whole routed MLP are compared in fp32 within the grouped-matmul tolerance."""
import pytest
import torch

import cabi
import oracle.ops_ref as R

pytestmark = pytest.mark.gpu
H = torch.float16


@pytest.mark.parametrize(
    "tokens,topk,E,invalid",
    [
        (4096, 8, 128, False),     # configs[3] routing
        (1000, 2, 8, True),        # n not a multiple of the slice, ids -1 and E mixed in
        (1, 1, 1, False),
        (128, 8, 128, True),       # 1024 ids: the largest table of the one-workgroup sort
        (205, 5, 128, True),       # 1025 ids: the sliced sort
        (8, 8, 4095, False),
        (100, 8, 4095, True),
        (63, 1, 2, False),
        (77, 6, 300, True),        # more experts than lanes of a wave
        (513, 1, 4095, False),     # largest expert count
        (20000, 4, 3, False),      # long runs of equal ids; more than 65536 ids: histogram, scan and scatter kernels
        (8192, 8, 255, True),      # 65536 ids, 256 buckets: the largest table of the two-launch sort
        (8193, 8, 255, True),      # one token more: the three-kernel sort
        (3000, 3, 256, True),      # 257 buckets: the three-kernel sort
        (1111, 7, 64, True),       # last workgroup with idle waves and a ragged last slice
    ],
)
def test_moe_sort_matches_a_stable_sort_exactly(dev, tokens, topk, E, invalid):
    import ascend910a_extras.moe as moe
    g = torch.Generator().manual_seed(tokens + E)
    ids = torch.randint(0, E, (tokens, topk), generator=g, dtype=torch.int32)
    if invalid:
        bad = torch.rand(tokens, topk, generator=g) < 0.1
        ids[bad] = -1
        ids[0, 0] = E
    s, inv, gl = moe.moe_sort(ids.to(dev), E)
    rs, rinv, rgl = R.moe_sort_ref(ids, E)
    assert torch.equal(gl.cpu(), rgl)
    assert torch.equal(s.cpu(), rs)
    assert torch.equal(inv.cpu(), rinv)
    assert s.dtype == torch.int32 and gl.dtype == torch.int64


def test_moe_sort_of_nothing(dev):
    import ascend910a_extras.moe as moe
    s, inv, gl = moe.moe_sort(torch.zeros(0, 4, dtype=torch.int32, device=dev), 16)
    assert s.numel() == 0 and torch.equal(gl.cpu(), torch.zeros(16, dtype=torch.int64))


def test_moe_gather_and_combine(dev):
    import ascend910a_extras.moe as moe
    g = torch.Generator().manual_seed(3)
    tokens, topk, E, hidden = 300, 4, 16, 256
    ids = torch.randint(0, E, (tokens, topk), generator=g, dtype=torch.int32)
    ids[torch.rand(tokens, topk, generator=g) < 0.15] = -1
    w = torch.rand(tokens, topk, generator=g)
    x = torch.randn(tokens, hidden, generator=g).half()
    s, inv, gl = moe.moe_sort(ids.to(dev), E)
    xs = moe.moe_gather(x.to(dev), s, gl, topk)
    end = int(gl[-1])
    assert end == int((ids >= 0).sum())
    assert torch.equal(xs.cpu()[:end], x[(s.cpu()[:end] // topk).long()])
    y = torch.randn(tokens * topk, hidden, generator=g).half()
    out = moe.moe_combine(y.to(dev), inv, w.to(dev), ids.to(dev), E)
    ref = torch.zeros(tokens, hidden)
    for t in range(tokens):
        for k in range(topk):
            if ids[t, k] >= 0:
                ref[t] += w[t, k] * y[int(inv[t * topk + k])].float()
    torch.testing.assert_close(out.cpu().float(), ref, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("tokens,topk,E,hidden,inter", [(512, 4, 16, 256, 128), (4096, 8, 128, 512, 256)])
def test_moe_mlp_end_to_end(dev, tokens, topk, E, hidden, inter):
    import ascend910a_extras.moe as moe
    g = torch.Generator().manual_seed(5)
    x = torch.randn(tokens, hidden, generator=g).half()
    logits = torch.randn(tokens, E, generator=g)
    wts, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
    wts = (wts / wts.sum(-1, keepdim=True)).float()
    ids = ids.int()
    w1 = (torch.randn(E, 2 * inter, hidden, generator=g) / hidden ** 0.5).half().transpose(1, 2)
    w2 = (torch.randn(E, hidden, inter, generator=g) / inter ** 0.5).half().transpose(1, 2)
    out = moe.moe_mlp(x.to(dev), ids.to(dev), wts.to(dev), w1.to(dev), w2.to(dev))
    ref = R.moe_mlp_ref(x, ids, wts, w1, w2)
    assert out.shape == (tokens, hidden) and out.dtype == H
    torch.testing.assert_close(out.cpu().float(), ref, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("tokens,topk,E,hidden,inter", [(700, 4, 16, 256, 128), (4096, 8, 128, 512, 384), (50, 2, 300, 384, 64),
                                                         # top-k that is not a power of two (the persistent kernel divides the
                                                         # flat index by it with a multiplication), enough rows per expert for it
                                                         (600, 3, 8, 256, 128), (500, 7, 16, 384, 64), (900, 5, 20, 256, 64),
                                                         (400, 6, 10, 512, 64), (300, 11, 12, 256, 64)])
def test_gather_fused_gate_up_equals_gather_then_matmul(dev, tokens, topk, E, hidden, inter):
    """The grouped matmul that reads its rows through the routing order against the explicit gather followed by the
    same kernel without the index: bit for bit (same arithmetic, same order), invalid ids included."""
    import ascend910a_extras.ascend910a_extras_C as C
    import ascend910a_extras.moe as moe
    g = torch.Generator().manual_seed(7)
    x = torch.randn(tokens, hidden, generator=g).half().to(dev)
    ids = torch.randint(0, E, (tokens, topk), generator=g, dtype=torch.int32)
    ids[torch.rand(tokens, topk, generator=g) < 0.05] = -1
    w1 = (torch.randn(E, 2 * inter, hidden, generator=g) / hidden ** 0.5).half().to(dev).transpose(1, 2)
    s, inv, gl = moe.moe_sort(ids.to(dev), E)
    end = int(gl[-1])
    a = C.grouped_matmul_swiglu_gather(x, s, topk, w1, gl)
    b = C.grouped_matmul_swiglu(moe.moe_gather(x, s, gl, topk), w1, gl)
    assert a.shape == (tokens * topk, inter)
    assert torch.equal(a[:end], b[:end])


@pytest.mark.parametrize("x_bytes", [(1 << 32) - (1 << 20), (1 << 32) + (1 << 22)])
def test_gather_fused_gate_up_reaches_rows_on_both_sides_of_4_gib(dev, x_bytes):
    """The persistent kernel addresses the gathered rows with 32-bit byte offsets, so an activation matrix of 4 GiB or
    more goes to the tile kernels instead: rows from the far end of x, just below and just above that size, against the
    explicit gather followed by the matmul."""
    import ascend910a_extras.ascend910a_extras_C as C
    hidden, inter, E, per = 2048, 128, 4, 256
    tokens = x_bytes // (2 * hidden)
    g = torch.Generator().manual_seed(11)
    x = torch.zeros(tokens, hidden, dtype=H, device=dev)
    picked = torch.cat([torch.randint(0, tokens, (E * per - 64,), generator=g), torch.arange(tokens - 64, tokens)])
    picked = picked[torch.randperm(E * per, generator=g)].to(torch.int32)
    rows = torch.randn(E * per, hidden, generator=g).half()
    x[picked.long().to(dev)] = rows.to(dev)      # duplicates in `picked`: the last write wins, both sides read x afterwards
    w1 = (torch.randn(E, 2 * inter, hidden, generator=g) / hidden ** 0.5).half().to(dev)   # [E, N, K]: the C ABI's layout
    gl = (torch.arange(1, E + 1, dtype=torch.int64) * per).to(dev)
    s = picked.to(dev)
    a = torch.empty(E * per, inter, dtype=H, device=dev)
    # through the C ABI: the Python operator insists on one index per (token, choice), the boundary does not
    assert cabi.lib().aops_grouped_matmul_swiglu_gather_f16(x.data_ptr(), s.data_ptr(), 1, tokens, w1.data_ptr(), gl.data_ptr(),
                                                            a.data_ptr(), E * per, hidden, E, 2 * inter, cabi.stream(dev)) == 0
    b = C.grouped_matmul_swiglu(x[s.long()], w1.transpose(1, 2), gl)
    torch.testing.assert_close(a.float(), b.float(), rtol=2e-2, atol=2e-2)
    assert float(a.float().abs().mean()) > 0.01


@pytest.mark.parametrize("tokens,topk,E,hidden,inter", [(50, 2, 300, 384, 64), (64, 8, 128, 512, 256), (8, 8, 16, 256, 128),
                                                         (300, 4, 32, 192, 96), (33, 2, 7, 64, 32)])
def test_decode_size_batches_take_the_small_tile_fused_kernels(dev, tokens, topk, E, hidden, inter):
    """Few rows per expert (and K that is not a multiple of 128): the fused entry points run small-tile kernels with the
    activation applied in the LDS staging of the epilogue and the row gather in the operand loads.  Against the chain
    of separate operators, against each other bit for bit, and against the oracle."""
    import ascend910a_extras.ascend910a_extras_C as C
    import ascend910a_extras.moe as moe
    g = torch.Generator().manual_seed(3)
    x = torch.randn(tokens, hidden, generator=g).half()
    ids = torch.randint(0, E, (tokens, topk), generator=g, dtype=torch.int32)
    ids[torch.rand(tokens, topk, generator=g) < 0.05] = -1
    w1 = (torch.randn(E, 2 * inter, hidden, generator=g) / hidden ** 0.5).half().transpose(1, 2)
    xd, w1d = x.to(dev), w1.to(dev)
    s, inv, gl = moe.moe_sort(ids.to(dev), E)
    end = int(gl[-1])
    xs = moe.moe_gather(xd, s, gl, topk)
    gathered = C.grouped_matmul_swiglu_gather(xd, s, topk, w1d, gl)
    fused_out = C.grouped_matmul_swiglu(xs, w1d, gl)
    chain = C.swiglu(C.grouped_matmul(xs, w1d, gl))
    assert gathered.shape == (tokens * topk, inter)
    assert torch.equal(fused_out[:end], gathered[:end])
    torch.testing.assert_close(fused_out[:end].float(), chain[:end].float(), rtol=2e-2, atol=2e-2)
    ref = R.swiglu_ref(R.grouped_matmul_ref(xs.cpu(), w1, gl.cpu()))
    torch.testing.assert_close(fused_out[:end].cpu().float(), ref[:end].float(), rtol=2e-2, atol=2e-2)
