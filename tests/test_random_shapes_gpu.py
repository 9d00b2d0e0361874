"""Seeded random shapes inside each operator's documented range, against the CPU oracle: the cases nobody
thought of writing down (odd group sizes, page sizes that are not powers of two, ragged batches, hidden
sizes that are multiples of 64 but of nothing larger)."""
import random

import pytest
import torch

import oracle.ops_ref as R

pytestmark = pytest.mark.gpu
H = torch.float16
TOL = dict(rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("seed", range(12))
def test_paged_attention_random_shape(ops, dev, seed):
    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    fast = seed % 2 == 0                                   # common shapes on even seeds, odd head and page sizes on odd
    D = 128 if fast else rnd.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256])
    P = rnd.choice([32, 64, 96, 128, 256]) if fast else rnd.choice([1, 4, 7, 16, 24, 48, 100, 128])
    group = rnd.choice([1, 2, 4, 8, 16]) if fast else rnd.choice([1, 2, 3, 5, 6, 7])
    Hkv = rnd.choice([1, 2, 3, 8])
    Hq = Hkv * group
    B = rnd.randint(1, 9)
    lens = [rnd.choice([0, 1, P - 1 if P > 1 else 1, P, P + 1, rnd.randint(1, 1500)]) for _ in range(B)]
    pages_per = [(l + P - 1) // P for l in lens]
    max_pages = max(max(pages_per), 1) + rnd.randint(0, 2)
    NB = sum(pages_per) + 3
    perm = torch.randperm(NB, generator=g)
    bt = torch.zeros(B, max_pages, dtype=torch.int32)
    c = 0
    for b, n in enumerate(pages_per):
        bt[b, :n] = perm[c:c + n].int()
        c += n
    kc = R.nz_pack(torch.randn(NB, P, Hkv, D, generator=g).half())
    vc = R.nz_pack(torch.randn(NB, P, Hkv, D, generator=g).half())
    q = torch.randn(B, Hq, D, generator=g).half()
    cl = torch.tensor(lens, dtype=torch.int32)
    o = ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), bt.to(dev), cl.to(dev)).cpu()
    ref = R.paged_attention_ref(q, kc, vc, bt, cl)
    torch.testing.assert_close(o.float(), ref.float(), **TOL)


@pytest.mark.parametrize("seed", range(10))
def test_paged_attention_random_batch(ops, dev, seed):
    """Batch sizes on either side of every switch of the launcher (a wave's 64 lanes, the ranking kernel, the plan
    kernel of the balanced partition), short sequences with a few long ones among them, tables wider than needed."""
    rnd = random.Random(100 + seed)
    g = torch.Generator().manual_seed(100 + seed)
    D = rnd.choice([64, 128, 128, 256, 80, 96, 192])
    P = rnd.choice([16, 64, 128])
    Hkv = rnd.choice([1, 2, 8])
    Hq = Hkv * rnd.choice([1, 4, 20])
    B = rnd.choice([rnd.randint(2, 20), rnd.randint(60, 70), rnd.randint(100, 300)])
    long_len = rnd.choice([700, 3000, 5000])
    lens = [rnd.choice([0, 1, 255, 256, 257, rnd.randint(1, 300)]) for _ in range(B)]
    for _ in range(rnd.randint(1, 3)):
        lens[rnd.randrange(B)] = rnd.randint(long_len // 2, long_len)
    pages_per = [(l + P - 1) // P for l in lens]
    max_pages = max(pages_per) + rnd.choice([0, 1, 40])
    NB = sum(pages_per) + 3
    perm = torch.randperm(NB, generator=g)
    bt = torch.full((B, max_pages), -1, dtype=torch.int32)
    c = 0
    for b, n in enumerate(pages_per):
        bt[b, :n] = perm[c:c + n].int()
        c += n
    kc = R.nz_pack(torch.randn(NB, P, Hkv, D, generator=g).half())
    vc = R.nz_pack(torch.randn(NB, P, Hkv, D, generator=g).half())
    q = torch.randn(B, Hq, D, generator=g).half()
    cl = torch.tensor(lens, dtype=torch.int32)
    o = ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), bt.to(dev), cl.to(dev)).cpu()
    ref = R.paged_attention_ref(q, kc, vc, bt.clamp(min=0), cl)
    torch.testing.assert_close(o.float(), ref.float(), **TOL)


@pytest.mark.parametrize("seed", range(8))
def test_token_operators_random_shape(ops, dev, seed):
    rnd = random.Random(100 + seed)
    g = torch.Generator().manual_seed(100 + seed)
    # add_rms_norm
    T, Hd = rnd.randint(1, 300), 64 * rnd.randint(1, 150)
    x = torch.randn(T, Hd, generator=g).half(); r = torch.randn(T, Hd, generator=g).half()
    w = (1 + 0.1 * torch.randn(Hd, generator=g)).half()
    eps = rnd.choice([1e-5, 1e-6])
    y, res = ops.add_rms_norm(x.to(dev), r.to(dev), w.to(dev), eps)
    y_ref, res_ref = R.add_rms_norm_ref(x, r, w, eps)
    assert torch.equal(res.cpu(), res_ref)
    torch.testing.assert_close(y.cpu().float(), y_ref.float(), **TOL)
    # swiglu
    T, d = rnd.randint(1, 500), 32 * rnd.randint(1, 200)
    xs = torch.randn(T, 2 * d, generator=g).half()
    torch.testing.assert_close(ops.swiglu(xs.to(dev)).cpu().float(), R.swiglu_ref(xs).float(), **TOL)
    # rope
    B, Hq, Hkv, D = rnd.randint(1, 40), rnd.randint(1, 40), rnd.randint(1, 9), 16 * rnd.randint(1, 16)
    maxpos = rnd.randint(1, 3000)
    q = torch.randn(B, Hq, D, generator=g).half(); k = torch.randn(B, Hkv, D, generator=g).half()
    cos, sin = R.build_cos_sin_cache(maxpos, D, theta=rnd.choice([1e4, 1e6]))
    pos = torch.randint(0, maxpos, (B,), generator=g).int()
    oq, ok = ops.rope(q.to(dev), k.to(dev), pos.to(dev), cos.to(dev), sin.to(dev))
    rq, rk = R.rope_ref(q, k, pos, cos, sin)
    torch.testing.assert_close(oq.cpu().float(), rq.float(), **TOL)
    torch.testing.assert_close(ok.cpu().float(), rk.float(), **TOL)
    # reshape_and_cache: bit-exact, some slots repeated out of range
    T, NB, P = rnd.randint(1, 200), rnd.randint(2, 30), rnd.choice([1, 8, 16, 33, 128])
    T = min(T, NB * P)
    key = torch.randn(T, Hkv, D, generator=g).half(); val = torch.randn(T, Hkv, D, generator=g).half()
    slots = torch.randperm(NB * P, generator=g)[:T].int()
    slots[rnd.randrange(T)] = rnd.choice([-1, NB * P, 2 ** 31 - 1])
    kc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half(); vc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()
    kcd, vcd = kc0.to(dev), vc0.to(dev)
    ops.reshape_and_cache(key.to(dev), val.to(dev), kcd, vcd, slots.to(dev))
    kc_ref, vc_ref = kc0.clone(), vc0.clone()
    R.reshape_and_cache_ref(key, kc_ref, slots, val, vc_ref)
    assert torch.equal(kcd.cpu(), kc_ref) and torch.equal(vcd.cpu(), vc_ref)


@pytest.mark.parametrize("seed", range(8))
def test_grouped_matmul_random_shape(ops, dev, seed):
    rnd = random.Random(200 + seed)
    g = torch.Generator().manual_seed(200 + seed)
    E = rnd.choice([1, 2, 7, 16, 65, 200])
    K, N = 64 * rnd.randint(1, 12), 64 * rnd.randint(1, 12)
    rows = rnd.randint(1, 3000)
    routed = rnd.randint(0, rows)
    ids = torch.randint(0, E, (routed,), generator=g)
    gl = R.make_group_list(ids, E)
    x = torch.randn(rows, K, generator=g).half()
    w = (torch.randn(E, N, K, generator=g) / K ** 0.5).half().transpose(1, 2)
    y = ops.grouped_matmul(x.to(dev), w.to(dev), gl.to(dev)).cpu()
    ref = R.grouped_matmul_ref(x, w, gl)
    torch.testing.assert_close(y[:routed].float(), ref[:routed].float(), rtol=2e-2, atol=2e-2)
