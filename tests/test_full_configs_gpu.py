"""The five BASELINE.json configurations at their full sizes on the GPU: against the CPU oracle
where the oracle finishes in seconds, and through size-independent properties (bit-exact
round trip, linearity, permutation invariance, checksums of disjoint parts) where it does not."""
import math

import pytest
import torch

import oracle.ops_ref as R

pytestmark = pytest.mark.gpu
H = torch.float16


def test_config1_add_rms_norm(ops, dev):
    torch.manual_seed(0)
    x = torch.randn(128, 4096).half(); r = torch.randn(128, 4096).half()
    w = (1 + 0.1 * torch.randn(4096)).half()
    y, res = ops.add_rms_norm(x.to(dev), r.to(dev), w.to(dev), 1e-6)
    y_ref, res_ref = R.add_rms_norm_ref(x, r, w, 1e-6)
    assert torch.equal(res.cpu(), res_ref)
    torch.testing.assert_close(y.cpu().float(), y_ref.float(), rtol=1e-2, atol=1e-2)
    # property: unit mean square before the weight
    ones = torch.ones(4096, dtype=H, device=dev)
    y1, _ = ops.add_rms_norm(x.to(dev), r.to(dev), ones, 1e-6)
    torch.testing.assert_close((y1.float() ** 2).mean(-1).cpu(), torch.ones(128), rtol=5e-3, atol=5e-3)


def test_config2_reshape_and_cache_roundtrip(ops, dev):
    torch.manual_seed(0)
    T, Hkv, D, NB, P = 2048, 8, 128, 1024, 128
    key = torch.randn(T, Hkv, D).half(); value = torch.randn(T, Hkv, D).half()
    slots = torch.randperm(NB * P)[:T].int()
    kc = torch.zeros(NB, Hkv * D // 16, P, 16, dtype=H, device=dev); vc = torch.zeros_like(kc)
    ops.reshape_and_cache(key.to(dev), value.to(dev), kc, vc, slots.to(dev))
    # bit-exact against the oracle
    kc_ref = torch.zeros(NB, Hkv * D // 16, P, 16, dtype=H); vc_ref = torch.zeros_like(kc_ref)
    R.reshape_and_cache_ref(key, kc_ref, slots, value, vc_ref)
    assert torch.equal(kc.cpu(), kc_ref) and torch.equal(vc.cpu(), vc_ref)
    # round trip: reading the written slots back returns the inputs, everything else is still zero
    dense = R.nz_unpack(kc.cpu(), Hkv).reshape(NB * P, Hkv, D)
    assert torch.equal(dense[slots.long()], key)
    assert int(torch.count_nonzero(dense)) == int(torch.count_nonzero(key))


def test_config3_dense_mlp(ops, dev):
    torch.manual_seed(0)
    bs, hidden, inter = 256, 4096, 14336
    x = torch.randn(bs, hidden).half()
    gu = torch.empty(2 * inter, hidden, dtype=H)
    for i in range(0, 2 * inter, 4096):
        gu[i:i + 4096] = (0.02 * torch.randn(min(4096, 2 * inter - i), hidden)).half()
    dn = (0.02 * torch.randn(hidden, inter)).half()
    gl = torch.tensor([bs], dtype=torch.int64, device=dev)
    h = ops.grouped_matmul(x.to(dev), gu.to(dev)[None].transpose(1, 2), gl)
    a = ops.swiglu(h)
    y = ops.grouped_matmul(a, dn.to(dev)[None].transpose(1, 2), gl)
    torch.testing.assert_close(a.cpu().float(), R.swiglu_ref(h.cpu()).float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(y.cpu().float(), R.mlp_ref(x, gu, dn).float(), rtol=2e-2, atol=2e-2)


def test_config4_moe_grouped_matmul(ops, dev):
    torch.manual_seed(0)
    E, hidden, inter, rows = 128, 2048, 768, 4096 * 8
    ids = torch.randint(0, E, (rows,))
    gl = R.make_group_list(ids, E)
    x = torch.randn(rows, hidden).half()
    w1 = torch.empty(E, 2 * inter, hidden, dtype=H)
    for e in range(E):
        w1[e] = (0.02 * torch.randn(2 * inter, hidden)).half()
    xd, wd, gd = x.to(dev), w1.to(dev), gl.to(dev)
    y = ops.grouped_matmul(xd, wd.transpose(1, 2), gd)
    # oracle on the first, a middle and the last expert (full rows of each)
    bounds = [0] + gl.tolist()
    yc = y.cpu()
    for e in (0, 1, 63, 127):
        s, t = bounds[e], bounds[e + 1]
        ref = (x[s:t].float() @ w1[e].float().T).half()
        torch.testing.assert_close(yc[s:t].float(), ref.float(), rtol=2e-2, atol=2e-2)
    # linearity in x over all 32768 rows: f(2x) == 2 f(x) exactly (power of two) wherever the
    # result is a normal fp16 number (subnormal results round on a fixed grid)
    y2 = ops.grouped_matmul(xd * 2, wd.transpose(1, 2), gd)
    normal = y.abs() >= 2.0 ** -13
    assert torch.equal(y2[normal], (y * 2)[normal])
    assert (y2.float() - 2 * y.float()).abs().max() <= 2.0 ** -23
    # negation: the matrix cores' internal accumulation is not exactly sign-symmetric, so the
    # results agree to the last fp16 bit or two rather than bit for bit
    yn = ops.grouped_matmul(-xd, wd.transpose(1, 2), gd)
    torch.testing.assert_close(yn.float(), -y.float(), rtol=2e-3, atol=1e-3)
    # routing invariance: a row's result depends only on its expert, not on its position in the group
    e = 5
    s, t = bounds[e], bounds[e + 1]
    perm = torch.randperm(t - s)
    xp = x.clone(); xp[s:t] = x[s:t][perm]
    yp = ops.grouped_matmul(xp.to(dev), wd.transpose(1, 2), gd).cpu()
    assert torch.equal(yp[s:t], yc[s:t][perm])
    assert torch.equal(yp[:s], yc[:s]) and torch.equal(yp[t:], yc[t:])
    # the second GEMM of the expert MLP (K = 768, N = 2048) against the oracle on the first, second, a middle
    # and the last expert, with the device's own activation as input ...
    hgu = ops.swiglu(y)
    hc = hgu.cpu()
    w2 = (0.02 * torch.randn(E, hidden, inter)).half()
    w2d = w2.to(dev)
    out = ops.grouped_matmul(hgu, w2d.transpose(1, 2), gd)
    outc = out.cpu()
    for e in (0, 1, 63, 127):
        s, t = bounds[e], bounds[e + 1]
        torch.testing.assert_close(hc[s:t].float(), R.swiglu_ref(yc[s:t]).float(), rtol=1e-2, atol=1e-2)
        ref = (hc[s:t].float() @ w2[e].float().T).half()
        torch.testing.assert_close(outc[s:t].float(), ref.float(), rtol=2e-2, atol=2e-2)
    # ... and end to end (oracle activation of the oracle's gate_up) on one expert
    s, t = bounds[127], bounds[128]
    ref = R.grouped_matmul_ref(R.swiglu_ref(R.grouped_matmul_ref(x[s:t], w1[127:128].transpose(1, 2), torch.tensor([t - s]))),
                               w2[127:128].transpose(1, 2), torch.tensor([t - s]))
    torch.testing.assert_close(outc[s:t].float(), ref.float(), rtol=2e-2, atol=2e-2)
    # the same size-independent properties for the down projection, over all 32768 rows
    out2 = ops.grouped_matmul(hgu * 2, w2d.transpose(1, 2), gd)
    normal = out.abs() >= 2.0 ** -13
    assert torch.equal(out2[normal], (out * 2)[normal])
    e = 77
    s, t = bounds[e], bounds[e + 1]
    perm = torch.randperm(t - s)
    hp = hc.clone(); hp[s:t] = hc[s:t][perm]
    outp = ops.grouped_matmul(hp.to(dev), w2d.transpose(1, 2), gd).cpu()
    assert torch.equal(outp[s:t], outc[s:t][perm])
    assert torch.equal(outp[:s], outc[:s]) and torch.equal(outp[t:], outc[t:])


def test_config4_every_expert_against_the_oracle(ops, dev):
    """Config 4 at full size, both projections, compared with the fp32 oracle on a seeded sample of rows from
    every one of the 128 experts (first row, last row and up to six more of each group: the rows where a
    scheduler or tile-boundary mistake would show)."""
    torch.manual_seed(1)
    E, hidden, inter, rows = 128, 2048, 768, 4096 * 8
    ids = torch.randint(0, E, (rows,))
    gl = R.make_group_list(ids, E)
    bounds = [0] + gl.tolist()
    x = torch.randn(rows, hidden).half()
    w1 = (0.02 * torch.randn(E, 2 * inter, hidden)).half()
    w2 = (0.02 * torch.randn(E, hidden, inter)).half()
    xd, gd = x.to(dev), gl.to(dev)
    y = ops.grouped_matmul(xd, w1.to(dev).transpose(1, 2), gd)
    h = ops.swiglu(y)
    out = ops.grouped_matmul(h, w2.to(dev).transpose(1, 2), gd)
    yc, hc, outc = y.cpu(), h.cpu(), out.cpu()
    g = torch.Generator().manual_seed(2)
    for e in range(E):
        s, t = bounds[e], bounds[e + 1]
        if t == s:
            continue
        pick = torch.unique(torch.cat([torch.tensor([s, t - 1]), s + torch.randint(0, t - s, (6,), generator=g)]))
        ref1 = x[pick].float() @ w1[e].float().T
        torch.testing.assert_close(yc[pick].float(), ref1, rtol=2e-2, atol=2e-2)
        ref2 = hc[pick].float() @ w2[e].float().T
        torch.testing.assert_close(outc[pick].float(), ref2, rtol=2e-2, atol=2e-2)


def test_config4_fused_gate_up_against_the_oracle(ops, dev):
    """The fused forms of config 4's gate_up projection at full size (K = 2048, N = 1536, 128 experts, 32768 routed
    rows) against the oracle chain swiglu_ref(grouped_matmul_ref(...)), not against the device's own chain:
    `fused.grouped_matmul_swiglu` on the expert-sorted rows and `grouped_matmul_swiglu_gather` on the token-order
    rows with the routing's sorted index, on sampled experts (whole groups) plus sampled rows of every expert."""
    import ascend910a_extras.ascend910a_extras_C as C
    import ascend910a_extras.fused as fused
    import ascend910a_extras.moe as moe

    torch.manual_seed(3)
    E, hidden, inter, tokens, topk = 128, 2048, 768, 4096, 8
    topk_ids = torch.randint(0, E, (tokens, topk), dtype=torch.int32)
    x = torch.randn(tokens, hidden).half()
    w1 = (0.02 * torch.randn(E, 2 * inter, hidden)).half()
    xd, w1d = x.to(dev), w1.to(dev)
    sorted_idx, _, gl = moe.moe_sort(topk_ids.to(dev), E)
    # the routing itself against the oracle's construction (benchmark/test_grouped_matmul.py:46-50)
    order_ref, _, gl_ref = R.moe_sort_ref(topk_ids, E)
    assert torch.equal(sorted_idx.cpu(), order_ref.int()) and torch.equal(gl.cpu(), gl_ref)
    bounds = [0] + gl_ref.tolist()
    src = (order_ref // topk).long()                 # token of every sorted row
    xs = x[src]                                      # expert-sorted activations, built on the host
    a_sorted = fused.grouped_matmul_swiglu(xs.to(dev), w1d.transpose(1, 2), gl).cpu()
    a_gather = C.grouped_matmul_swiglu_gather(xd, sorted_idx, topk, w1d.transpose(1, 2), gl).cpu()
    assert a_sorted.shape == (tokens * topk, inter)

    def oracle(rows_idx, e):
        n = len(rows_idx)
        return R.swiglu_ref(R.grouped_matmul_ref(xs[rows_idx], w1[e:e + 1].transpose(1, 2), torch.tensor([n])))

    for e in (0, 1, 64, 127):                         # whole groups
        s, t = bounds[e], bounds[e + 1]
        ref = oracle(torch.arange(s, t), e).float()
        torch.testing.assert_close(a_sorted[s:t].float(), ref, rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(a_gather[s:t].float(), ref, rtol=2e-2, atol=2e-2)
    g = torch.Generator().manual_seed(4)
    for e in range(E):                                # first, last and four more rows of every expert
        s, t = bounds[e], bounds[e + 1]
        if t == s:
            continue
        pick = torch.unique(torch.cat([torch.tensor([s, t - 1]), s + torch.randint(0, t - s, (4,), generator=g)]))
        ref = oracle(pick, e).float()
        torch.testing.assert_close(a_sorted[pick].float(), ref, rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(a_gather[pick].float(), ref, rtol=2e-2, atol=2e-2)


def test_config5_decode_attention_with_rope(ops, dev):
    torch.manual_seed(0)
    B, Hq, Hkv, D, P, NB = 64, 32, 8, 128, 128, 2304
    ctx = torch.randint(512, 4097, (B,), dtype=torch.int32)
    perm = torch.randperm(NB)
    bt = torch.zeros(B, 32, dtype=torch.int32)
    c = 0
    for b in range(B):
        npg = (int(ctx[b]) + P - 1) // P
        bt[b, :npg] = perm[c:c + npg].int(); c += npg
    kc = torch.empty(NB, Hkv * D // 16, P, 16, dtype=H); vc = torch.empty_like(kc)
    for i in range(0, NB, 256):
        kc[i:i + 256] = torch.randn(min(256, NB - i), Hkv * D // 16, P, 16).half()
        vc[i:i + 256] = torch.randn(min(256, NB - i), Hkv * D // 16, P, 16).half()
    q = torch.randn(B, Hq, D).half(); k = torch.randn(B, Hkv, D).half(); v = torch.randn(B, Hkv, D).half()
    cos, sin = R.build_cos_sin_cache(4096, D, theta=1e6)
    pos = (ctx - 1).int()
    slots = torch.tensor([int(bt[b, int(pos[b]) // P]) * P + int(pos[b]) % P for b in range(B)], dtype=torch.int32)
    kcd, vcd, btd, ctxd = kc.to(dev), vc.to(dev), bt.to(dev), ctx.to(dev)
    oq, ok = ops.rope(q.to(dev), k.to(dev), pos.to(dev), cos.to(dev), sin.to(dev))
    ops.reshape_and_cache(ok, v.to(dev), kcd, vcd, slots.to(dev))
    o = ops.paged_attention(oq, kcd, vcd, btd, ctxd)
    # oracle, stage by stage on the whole batch.  rope: fp32 math on both sides, but the GPU may
    # contract a*c - b*s into a fused multiply-add, so the last bit can differ
    rq, rk = R.rope_ref(q, k, pos, cos, sin)
    torch.testing.assert_close(oq.cpu().float(), rq.float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(ok.cpu().float(), rk.float(), rtol=1e-2, atol=1e-2)
    # cache write: bit-exact for what the device's own rope produced
    R.reshape_and_cache_ref(ok.cpu(), kc, slots, v, vc)
    assert torch.equal(kcd.cpu(), kc) and torch.equal(vcd.cpu(), vc)
    ref = R.paged_attention_ref(oq.cpu(), kc, vc, bt, ctx)
    torch.testing.assert_close(o.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)
    assert (o.cpu().float() - ref.float()).abs().max() < 2e-3
    # permuting the physical pages together with the tables changes nothing, bit for bit
    p2 = torch.randperm(NB)
    inv = torch.empty_like(p2); inv[p2] = torch.arange(NB)
    o2 = ops.paged_attention(oq, kcd[p2.to(dev)], vcd[p2.to(dev)], inv[bt.long()].int().to(dev), ctxd)
    assert torch.equal(o2, o)
    # permuting the sequences of the batch permutes the outputs, bit for bit
    pb = torch.randperm(B)
    o3 = ops.paged_attention(oq[pb.to(dev)], kcd, vcd, btd[pb.to(dev)], ctxd[pb.to(dev)])
    assert torch.equal(o3, o[pb.to(dev)])
