"""Every entry point enqueues on the caller's stream without synchronising or reading device data on
the host (block tables, context lengths, slots and group_list stay on the device), so a whole decode
step plus an expert MLP can be captured in one HIP graph.  The graph is replayed several times with the
inputs changed in place between replays, with eager work and synchronisations in between, and every
replay is compared with the eager result for the same inputs."""
import pytest
import torch

import oracle.ops_ref as R

pytestmark = pytest.mark.gpu
H = torch.float16


def test_decode_step_and_expert_mlp_in_one_graph(ops, dev):
    import ascend910a_extras.fused as fused

    g = torch.Generator().manual_seed(9)
    B, Hq, Hkv, D, P, NB, maxp = 8, 32, 8, 128, 128, 80, 8
    E, K, I, rows = 16, 256, 256, 2048

    def new_inputs(seed):
        gg = torch.Generator().manual_seed(seed)
        ctx = torch.randint(1, P * maxp + 1, (B,), generator=gg, dtype=torch.int32)
        perm = torch.randperm(NB, generator=gg)
        bt = torch.zeros(B, maxp, dtype=torch.int32)
        c = 0
        for b in range(B):
            npg = (int(ctx[b]) + P - 1) // P
            bt[b, :npg] = perm[c:c + npg].int()
            c += npg
        pos = (ctx - 1).int()
        slots = torch.tensor([int(bt[b, int(pos[b]) // P]) * P + int(pos[b]) % P for b in range(B)], dtype=torch.int32)
        ids = torch.randint(0, E, (rows,), generator=gg)
        return dict(
            q=torch.randn(B, Hq, D, generator=gg).half(), k=torch.randn(B, Hkv, D, generator=gg).half(),
            v=torch.randn(B, Hkv, D, generator=gg).half(), pos=pos, slots=slots, bt=bt, ctx=ctx,
            x=torch.randn(B, 512, generator=gg).half(), r=torch.randn(B, 512, generator=gg).half(),
            xs=torch.randn(rows, K, generator=gg).half(), gl=R.make_group_list(ids, E),
        )

    cos, sin = R.build_cos_sin_cache(P * maxp, D, theta=1e6)
    cosd, sind = cos.to(dev), sin.to(dev)
    wn = (1 + 0.1 * torch.randn(512, generator=g)).half().to(dev)
    w1 = (0.05 * torch.randn(E, 2 * I, K, generator=g)).half().to(dev).transpose(1, 2)
    w2 = (0.05 * torch.randn(E, K, I, generator=g)).half().to(dev).transpose(1, 2)
    kc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half().to(dev)
    vc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half().to(dev)

    static = {k: v.to(dev) for k, v in new_inputs(0).items()}
    kc, vc = kc0.clone(), vc0.clone()

    def step():
        y, res = ops.add_rms_norm(static["x"], static["r"], wn, 1e-6)
        oq, ok = ops.rope(static["q"], static["k"], static["pos"], cosd, sind)
        ops.reshape_and_cache(ok, static["v"], kc, vc, static["slots"])
        o = ops.paged_attention(oq, kc, vc, static["bt"], static["ctx"])
        oq2 = fused.rope_reshape_and_cache(static["q"], static["k"], static["v"], static["pos"], cosd, sind, kc, vc,
                                           static["slots"])
        h = ops.swiglu(ops.grouped_matmul(static["xs"], w1, static["gl"]))
        hf = fused.grouped_matmul_swiglu(static["xs"], w1, static["gl"])
        out = ops.grouped_matmul(h, w2, static["gl"])
        return [y, res, oq, ok, o, oq2, h, hf, out]

    # warm-up on a side stream (one-time kernel attribute set-up happens outside the capture)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()

    for seed in (1, 2, 3, 4):
        fresh = new_inputs(seed)
        for name, t in fresh.items():
            static[name].copy_(t.to(dev))
        kc.copy_(kc0); vc.copy_(vc0)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        got_kc, got_vc = kc.clone(), vc.clone()
        # eager, same inputs, fresh caches
        kc.copy_(kc0); vc.copy_(vc0)
        want = step()
        torch.cuda.synchronize()
        end = int(fresh["gl"][-1])
        for i, (a, b) in enumerate(zip(got, want)):
            if i >= 6:   # grouped matmul outputs: rows past the last group are never written
                a, b = a[:end], b[:end]
            assert torch.equal(a, b), f"replay with seed {seed}: output {i} differs from the eager call"
        assert torch.equal(got_kc, kc) and torch.equal(got_vc, vc)
    # and the eager results themselves are right (attention of the last seed against the oracle)
    ref = R.paged_attention_ref(want[2].cpu(), kc.cpu(), vc.cpu(), fresh["bt"], fresh["ctx"])
    torch.testing.assert_close(want[4].cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("B,maxp", [(100, 40), (100, 8), (12, 40)])
def test_paged_attention_launch_forms_in_a_graph(ops, dev, B, maxp):
    """The partition of the work is computed on the device at every replay, not at capture: batches of 100
    sequences with a block table of 5120 tokens (plan kernel + balanced shares + merge) or of 1024 tokens
    (ranking kernel + whole sequences) and a small batch (in-wave partition), replayed with other context
    lengths and block tables and compared with the oracle each time."""
    Hq, Hkv, D, P = 8, 2, 128, 128
    NB = B * maxp + 4
    g = torch.Generator().manual_seed(B + maxp)
    kc_h = R.nz_pack(torch.randn(NB, P, Hkv, D, generator=g).half())
    vc_h = R.nz_pack(torch.randn(NB, P, Hkv, D, generator=g).half())
    kc, vc = kc_h.to(dev), vc_h.to(dev)

    def new_inputs(seed):
        gg = torch.Generator().manual_seed(seed)
        ctx = torch.randint(0, 300, (B,), generator=gg, dtype=torch.int32)
        ctx[seed % B] = P * maxp                       # one sequence fills its table row
        ctx[(seed * 7 + 3) % B] = P * maxp // 2 + 1
        bt = torch.randperm(NB, generator=gg)[:B * maxp].int().reshape(B, maxp)
        return torch.randn(B, Hq, D, generator=gg).half(), bt, ctx

    q0, bt0, ctx0 = new_inputs(0)
    q, bt, ctx = q0.to(dev), bt0.to(dev), ctx0.to(dev)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        ops.paged_attention(q, kc, vc, bt, ctx)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o = ops.paged_attention(q, kc, vc, bt, ctx)
    for seed in (1, 2, 3):
        qh, bth, ctxh = new_inputs(seed)
        q.copy_(qh.to(dev)); bt.copy_(bth.to(dev)); ctx.copy_(ctxh.to(dev))
        graph.replay()
        torch.cuda.synchronize()
        ref = R.paged_attention_ref(qh, kc_h, vc_h, bth, ctxh)
        torch.testing.assert_close(o.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)
        assert torch.equal(o, ops.paged_attention(q, kc, vc, bt, ctx)), f"replay {seed} differs from the eager call"


def test_two_streams_concurrently(ops, dev):
    """Entry points keep no device-side state between calls, so independent work on two streams may overlap:
    a grouped matmul chain on one stream and decode attention on the other, several rounds, against the same
    work done alone."""
    import ascend910a_extras.fused as fused

    g = torch.Generator().manual_seed(21)
    E, K, I, rows = 32, 512, 256, 8192
    xs = torch.randn(rows, K, generator=g).half().to(dev)
    w1 = (0.05 * torch.randn(E, 2 * I, K, generator=g)).half().to(dev).transpose(1, 2)
    gl = R.make_group_list(torch.randint(0, E, (rows,), generator=g), E).to(dev)
    B, Hq, Hkv, D, P, NB = 16, 32, 8, 128, 128, 160
    kc = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half().to(dev)
    vc = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half().to(dev)
    bt = torch.randperm(NB, generator=g).int().reshape(B, NB // B).to(dev)
    cl = torch.randint(1, P * (NB // B) + 1, (B,), generator=g, dtype=torch.int32).to(dev)
    q = torch.randn(B, Hq, D, generator=g).half().to(dev)
    want_h = fused.grouped_matmul_swiglu(xs, w1, gl)
    want_o = ops.paged_attention(q, kc, vc, bt, cl)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(5):
        with torch.cuda.stream(s1):
            h = fused.grouped_matmul_swiglu(xs, w1, gl)
            h2 = ops.swiglu(ops.grouped_matmul(xs, w1, gl))
        with torch.cuda.stream(s2):
            o = ops.paged_attention(q, kc, vc, bt, cl)
            o2 = ops.paged_attention(q, kc, vc, bt, cl)
        torch.cuda.synchronize()
        assert torch.equal(h, want_h) and torch.equal(o, want_o) and torch.equal(o2, want_o)
        torch.testing.assert_close(h2.float(), want_h.float(), rtol=2e-2, atol=2e-2)
