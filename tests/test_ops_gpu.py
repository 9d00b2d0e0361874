"""GPU parity tests: every operator, called through the Python API (and so through the C ABI
of libaops.so), against the CPU oracle on the same seeded inputs.

Bars (from the project's statement of parity): reshape_and_cache bit-exact; fp16 operators
within rtol = atol = 1e-2 of the fp32 oracle; grouped_matmul within rtol = atol = 2e-2."""
import math

import pytest
import torch

import cabi
import oracle.ops_ref as R

pytestmark = pytest.mark.gpu
H = torch.float16
TOL = dict(rtol=1e-2, atol=1e-2)
GMM_TOL = dict(rtol=2e-2, atol=2e-2)


def _gen(seed):
    return torch.Generator().manual_seed(seed)


# ----------------------------------------------------------------------------- add_rms_norm
@pytest.mark.parametrize(
    "T,Hd,eps",
    [(128, 4096, 1e-6), (1024, 1024, 1e-6), (1, 64, 1e-5), (7, 192, 1e-6), (3, 8192, 1e-6),
     (2, 16384, 1e-6), (2, 65536, 1e-6), (2, 65536 + 64, 1e-6), (4096, 4096, 1e-6), (0, 128, 1e-6)],
)
def test_add_rms_norm(ops, dev, T, Hd, eps):
    g = _gen(0)
    x = torch.randn(T, Hd, generator=g).half()
    r = torch.randn(T, Hd, generator=g).half()
    w = (1 + 0.1 * torch.randn(Hd, generator=g)).half()
    y_ref, res_ref = R.add_rms_norm_ref(x, r, w, eps)
    xd, rd = x.to(dev), r.to(dev)
    y, res = ops.add_rms_norm(xd, rd, w.to(dev), eps)
    torch.cuda.synchronize()
    assert y.shape == (T, Hd) and y.dtype == H
    assert torch.equal(res.cpu(), res_ref)  # fp16 sum is exactly determined
    torch.testing.assert_close(y.cpu().float(), y_ref.float(), **TOL)
    assert torch.equal(xd.cpu(), x) and torch.equal(rd.cpu(), r)  # inputs untouched


def test_add_rms_norm_default_epsilon_and_reference_script_shape(ops, dev):
    # benchmark/test_add_rms_norm.py:14-22: T=1024, dim=1024, weight ~ N(0,1); its tolerance is 1e-3
    g = _gen(0)
    x = torch.randn(1024, 1024, generator=g).half()
    r = torch.randn(1024, 1024, generator=g).half()
    w = torch.randn(1024, generator=g).half()
    y_ref, res_ref = R.add_rms_norm_ref(x, r, w, 1e-6)
    y, res = ops.add_rms_norm(x.to(dev), r.to(dev), w.to(dev), 1e-6)
    torch.testing.assert_close(y.cpu(), y_ref, atol=4e-3, rtol=4e-3)
    torch.testing.assert_close(res.cpu(), res_ref, atol=1e-3, rtol=1e-3)
    y5, _ = ops.add_rms_norm(x.to(dev), r.to(dev), w.to(dev))  # epsilon defaults to 1e-5
    y5_ref, _ = R.add_rms_norm_ref(x, r, w, 1e-5)
    torch.testing.assert_close(y5.cpu().float(), y5_ref.float(), **TOL)


# ----------------------------------------------------------------------------- swiglu
@pytest.mark.parametrize("T,d", [(256, 14336), (2048, 192), (32768, 768), (1, 32), (5, 96), (3, 4000), (0, 64)])
def test_swiglu(ops, dev, T, d):
    x = torch.randn(T, 2 * d, generator=_gen(0)).half()
    if T > 0:
        x[0, :8] = torch.tensor([0.0, -0.0, 20.0, -20.0, 65504.0, -65504.0, 1e-4, -1e-4]).half()
    y = ops.swiglu(x.to(dev))
    assert y.shape == (T, d)
    torch.testing.assert_close(y.cpu().float(), R.swiglu_ref(x).float(), **TOL)


# ----------------------------------------------------------------------------- rope
@pytest.mark.parametrize("B,Hq,Hkv,D,max_pos", [(64, 32, 8, 128, 4096), (4, 32, 8, 128, 40960), (1, 1, 1, 16, 8), (3, 5, 5, 64, 100), (2, 16, 2, 256, 64)])
def test_rope(ops, dev, B, Hq, Hkv, D, max_pos):
    g = _gen(0)
    q = torch.randn(B, Hq, D, generator=g).half()
    k = torch.randn(B, Hkv, D, generator=g).half()
    cos, sin = R.build_cos_sin_cache(max_pos, D, theta=1e6)
    pos = torch.randint(0, max_pos, (B,), generator=g, dtype=torch.int32)
    pos[0] = 0
    pos[-1] = max_pos - 1
    out = ops.rope(q.to(dev), k.to(dev), pos.to(dev), cos.to(dev), sin.to(dev))
    assert isinstance(out, (list, tuple)) and len(out) == 2
    rq, rk = R.rope_ref(q, k, pos, cos, sin)
    torch.testing.assert_close(out[0].cpu().float(), rq.float(), **TOL)
    torch.testing.assert_close(out[1].cpu().float(), rk.float(), **TOL)
    if B > 1:
        assert torch.equal(out[0][0].cpu(), q[0])  # position 0 is the identity, exactly
    # native-fp16 evaluation of the reference formula also agrees within tolerance
    nq, _ = R.rope_ref(q, k, pos, cos, sin, compute_dtype=H)
    torch.testing.assert_close(out[0].cpu().float(), nq.float(), **TOL)


# ----------------------------------------------------------------------------- reshape_and_cache
def test_reshape_and_cache_reference_known_answer(ops, dev):
    """benchmark/test_reshape_and_cache.py:29-84 on the GPU, both of its cases, bit-exact."""
    torch.manual_seed(42)
    slots = torch.tensor([6, 134, 212, 290], dtype=torch.int32)
    key = torch.randn(4, 8, 128, dtype=H)
    value = torch.randn(4, 8, 128, dtype=H)
    kc_ref = torch.zeros(583, 64, 128, 16, dtype=H); vc_ref = torch.zeros_like(kc_ref)
    R.reshape_and_cache_ref(key, kc_ref, slots, value, vc_ref)
    kc = torch.zeros_like(kc_ref, device=dev); vc = torch.zeros_like(kc_ref, device=dev)
    assert ops.reshape_and_cache(key.to(dev), value.to(dev), kc, vc, slots.to(dev)) is None
    assert torch.equal(kc.cpu(), kc_ref) and torch.equal(vc.cpu(), vc_ref)
    key2 = torch.randn(4, 8, 128, dtype=H)
    kc2_ref = torch.zeros_like(kc_ref)
    R.reshape_and_cache_ref(key2, kc2_ref, slots)
    kc2 = torch.zeros_like(kc_ref, device=dev); vc2 = torch.zeros_like(kc_ref, device=dev)
    ops.reshape_and_cache(key2.to(dev), None, kc2, None, slots.to(dev))
    assert torch.equal(kc2.cpu(), kc2_ref)
    assert torch.count_nonzero(vc2) == 0


def test_reshape_and_cache_golden_fixture(ops, dev):
    """Committed fixture (tests/golden/reshape_and_cache_kat.npz): the reference's inputs bit for
    bit, the expected cache given as explicit flat positions."""
    import os

    import numpy as np

    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reshape_and_cache_kat.npz"))
    as_half = lambda a: torch.from_numpy(a.copy()).view(H)
    key, value, key2 = as_half(d["key_bits"]), as_half(d["value_bits"]), as_half(d["key2_bits"])
    slots = torch.from_numpy(d["slots"].copy())
    shape = tuple(int(v) for v in d["cache_shape"])
    idx = torch.from_numpy(d["flat_index"].reshape(-1))
    kc = torch.zeros(shape, dtype=H, device=dev); vc = torch.zeros(shape, dtype=H, device=dev)
    ops.reshape_and_cache(key.to(dev), value.to(dev), kc, vc, slots.to(dev))
    want_k = torch.zeros(kc.numel(), dtype=H); want_v = torch.zeros_like(want_k)
    want_k[idx] = key.reshape(-1); want_v[idx] = value.reshape(-1)
    assert torch.equal(kc.cpu().reshape(-1), want_k) and torch.equal(vc.cpu().reshape(-1), want_v)
    kc.zero_(); vc.zero_()
    ops.reshape_and_cache(key2.to(dev), None, kc, None, slots.to(dev))  # key-only case of the reference
    want_k.zero_(); want_k[idx] = key2.reshape(-1)
    assert torch.equal(kc.cpu().reshape(-1), want_k) and torch.count_nonzero(vc) == 0


@pytest.mark.parametrize("T,Hkv,D,NB,P", [(2048, 8, 128, 1024, 128), (64, 8, 128, 40, 128), (17, 2, 64, 9, 16), (5, 1, 16, 3, 7), (0, 8, 128, 4, 128)])
def test_reshape_and_cache_bit_exact(ops, dev, T, Hkv, D, NB, P):
    g = _gen(0)
    key = torch.randn(T, Hkv, D, generator=g).half()
    value = torch.randn(T, Hkv, D, generator=g).half()
    slots = torch.randperm(NB * P, generator=g)[:T].int()
    base_k = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()  # pre-existing cache contents
    base_v = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()
    kc_ref, vc_ref = base_k.clone(), base_v.clone()
    R.reshape_and_cache_ref(key, kc_ref, slots, value, vc_ref)
    kc, vc = base_k.to(dev), base_v.to(dev)
    ops.reshape_and_cache(key.to(dev), value.to(dev), kc, vc, slots.to(dev))
    # bit-exact including -0.0 / NaN payloads: compare the raw 16-bit patterns
    assert torch.equal(kc.cpu().view(torch.int16), kc_ref.view(torch.int16))
    assert torch.equal(vc.cpu().view(torch.int16), vc_ref.view(torch.int16))


def test_reshape_and_cache_skips_bad_slots_and_roundtrips(ops, dev):
    g = _gen(1)
    NB, P, Hkv, D = 6, 32, 4, 128
    dense = torch.randn(NB, P, Hkv, D, generator=g).half()
    slots = torch.randperm(NB * P, generator=g).int()
    key = dense.reshape(NB * P, Hkv, D)[slots.long()]
    kc = torch.zeros(NB, Hkv * D // 16, P, 16, dtype=H, device=dev)
    ops.reshape_and_cache(key.to(dev), None, kc, None, slots.to(dev))
    assert torch.equal(kc.cpu(), R.nz_pack(dense))  # filling every slot == packing the dense tensor
    kc.zero_()
    bad = torch.tensor([-1, NB * P, 2**31 - 1, -(2**31), 5], dtype=torch.int32)
    ops.reshape_and_cache(key[:5].to(dev), key[:5].to(dev), kc, kc.clone(), bad.to(dev))
    got = kc.cpu()
    assert torch.equal(got[0, :, 5, :].reshape(-1), key[4].reshape(-1))
    got[0, :, 5, :] = 0
    assert torch.count_nonzero(got) == 0


@pytest.mark.parametrize("B,Hq,Hkv,D,NB,P", [(64, 32, 8, 128, 2304, 128), (5, 6, 2, 64, 7, 16), (3, 1, 1, 16, 4, 8), (17, 16, 16, 256, 9, 32),
                                             (700, 8, 2, 128, 16, 64)])   # prefill-sized: more than 256 workgroups
def test_rope_reshape_and_cache_fused_equals_the_chain(ops, dev, B, Hq, Hkv, D, NB, P):
    """One launch against rope -> reshape_and_cache: q, k and both caches bit for bit, including a slot that is
    out of range (skipped by both) and cache contents that must stay untouched; and against the oracle."""
    import ascend910a_extras.fused as fused
    g = _gen(5)
    q = torch.randn(B, Hq, D, generator=g).half()
    k = torch.randn(B, Hkv, D, generator=g).half()
    v = torch.randn(B, Hkv, D, generator=g).half()
    cos, sin = R.build_cos_sin_cache(512, D, theta=1e6)
    pos = torch.randint(0, 512, (B,), generator=g).int()
    slots = torch.randperm(NB * P, generator=g)[:B].int()
    slots[B // 2] = NB * P + 3          # skipped
    kc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()
    vc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()
    qd, kd, vd, posd, cosd, sind, sld = (t.to(dev) for t in (q, k, v, pos, cos, sin, slots))
    kc_a, vc_a = kc0.to(dev), vc0.to(dev)
    oq_a, ok_a = ops.rope(qd, kd, posd, cosd, sind)
    ops.reshape_and_cache(ok_a, vd, kc_a, vc_a, sld)
    kc_b, vc_b = kc0.to(dev), vc0.to(dev)
    oq_b, ok_b = fused.rope_reshape_and_cache(qd, kd, vd, posd, cosd, sind, kc_b, vc_b, sld, return_k=True)
    assert torch.equal(oq_a, oq_b) and torch.equal(ok_a, ok_b)
    assert torch.equal(kc_a, kc_b) and torch.equal(vc_a, vc_b)
    kc_c, vc_c = kc0.to(dev), vc0.to(dev)
    oq_c = fused.rope_reshape_and_cache(qd, kd, vd, posd, cosd, sind, kc_c, vc_c, sld)
    assert torch.equal(oq_c, oq_a) and torch.equal(kc_c, kc_a) and torch.equal(vc_c, vc_a)
    # oracle: rotation within tolerance; the cache holds exactly what the device rotation produced
    rq, rk = R.rope_ref(q, k, pos, cos, sin)
    torch.testing.assert_close(oq_b.cpu().float(), rq.float(), **TOL)
    torch.testing.assert_close(ok_b.cpu().float(), rk.float(), **TOL)
    kc_ref, vc_ref = kc0.clone(), vc0.clone()
    R.reshape_and_cache_ref(ok_b.cpu(), kc_ref, slots, v, vc_ref)
    assert torch.equal(kc_b.cpu(), kc_ref) and torch.equal(vc_b.cpu(), vc_ref)


@pytest.mark.parametrize("B,Hq,Hkv,D,NB,P", [(64, 32, 8, 128, 2304, 128), (5, 6, 2, 64, 7, 16), (3, 1, 1, 16, 4, 8), (9, 4, 4, 256, 9, 32), (7, 3, 1, 32, 5, 4),
                                             (1200, 4, 4, 64, 80, 16),
                                             # head sizes whose threads per head are no power of two: 3, 5, 6, 7, 10, 12 and 20 threads
                                             (37, 5, 1, 48, 9, 16), (300, 7, 3, 80, 40, 8), (11, 4, 2, 96, 5, 16), (5, 3, 1, 112, 4, 4),
                                             (19, 9, 3, 160, 7, 16), (64, 16, 4, 192, 20, 32), (3, 2, 2, 320, 3, 16)])
def test_qknorm_rope_reshape_and_cache_fused(ops, dev, B, Hq, Hkv, D, NB, P):
    """Per-head RMSNorm of q and k + rope + cache write in one launch, against the oracle (RMSNorm rounded to fp16,
    then rotated) and against the chain of separate device operators where those take the shape."""
    import ascend910a_extras.fused as fused
    g = _gen(8)
    q = torch.randn(B, Hq, D, generator=g).half()
    k = torch.randn(B, Hkv, D, generator=g).half()
    v = torch.randn(B, Hkv, D, generator=g).half()
    wq = (1 + 0.2 * torch.randn(D, generator=g)).half()
    wk = (1 + 0.2 * torch.randn(D, generator=g)).half()
    eps = 1e-6
    cos, sin = R.build_cos_sin_cache(512, D, theta=1e6)
    pos = torch.randint(0, 512, (B,), generator=g).int()
    slots = torch.randperm(NB * P, generator=g)[:B].int()
    kc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()
    vc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()
    qd, kd, vd, posd, cosd, sind, sld = (t.to(dev) for t in (q, k, v, pos, cos, sin, slots))
    kcd, vcd = kc0.to(dev), vc0.to(dev)
    oq, ok = fused.rope_reshape_and_cache(qd, kd, vd, posd, cosd, sind, kcd, vcd, sld, return_k=True,
                                          q_norm_weight=wq.to(dev), k_norm_weight=wk.to(dev), epsilon=eps)

    def rms(t, w):
        t = t.float()
        return (t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w.float()).half()

    rq, rk = R.rope_ref(rms(q, wq), rms(k, wk), pos, cos, sin)
    torch.testing.assert_close(oq.cpu().float(), rq.float(), **TOL)
    torch.testing.assert_close(ok.cpu().float(), rk.float(), **TOL)
    # the caches hold exactly the rotated k the kernel reports, and v untouched
    kc_ref, vc_ref = kc0.clone(), vc0.clone()
    R.reshape_and_cache_ref(ok.cpu(), kc_ref, slots, v, vc_ref)
    assert torch.equal(kcd.cpu(), kc_ref) and torch.equal(vcd.cpu(), vc_ref)
    if D % 64 == 0:   # the separate RMSNorm operator takes rows that are multiples of 64
        zq = torch.zeros(B * Hq, D, dtype=H, device=dev); zk = torch.zeros(B * Hkv, D, dtype=H, device=dev)
        qn = ops.add_rms_norm(qd.view(B * Hq, D), zq, wq.to(dev), eps)[0].view(B, Hq, D)
        kn = ops.add_rms_norm(kd.view(B * Hkv, D), zk, wk.to(dev), eps)[0].view(B, Hkv, D)
        cq, ck = ops.rope(qn, kn, posd, cosd, sind)
        torch.testing.assert_close(oq.float(), cq.float(), rtol=2e-3, atol=2e-3)
        torch.testing.assert_close(ok.float(), ck.float(), rtol=2e-3, atol=2e-3)


# ----------------------------------------------------------------------------- grouped_matmul
def _gmm_case(rows, K, N, E, seed, counts=None, wstd=0.02):
    g = _gen(seed)
    x = torch.randn(rows, K, generator=g).half()
    w = (wstd * torch.randn(E, N, K, generator=g)).half().transpose(1, 2)
    if counts is None:
        ids = torch.randint(0, E, (rows,), generator=g)
        gl = R.make_group_list(ids, E)
    else:
        gl = torch.tensor(counts).cumsum(0).to(torch.int64)
    return x, w, gl


@pytest.mark.parametrize(
    "rows,K,N,E,counts",
    [
        (1024, 256, 256, 8, None),
        (300, 64, 64, 4, [0, 1, 170, 129]),        # empty group, single row, >1 tile, minimum K and N
        (513, 128, 192, 3, [128, 256, 100]),        # exact tile, two tiles, rows past the last group
        (96, 2048, 1536, 1, [96]),                  # E = 1: plain GEMM
        (700, 768, 2048, 5, [0, 0, 700, 0, 0]),     # everything in one expert
        (64, 512, 64, 130, None),                   # more experts than lanes in a wave
    ],
)
def test_grouped_matmul(ops, dev, rows, K, N, E, counts):
    x, w, gl = _gmm_case(rows, K, N, E, seed=0, counts=counts)
    sentinel = 77.0
    ref = R.grouped_matmul_ref(x, w, gl, out=torch.full((rows, N), sentinel).half())
    y = ops.grouped_matmul(x.to(dev), w.to(dev), gl.to(dev))
    assert y.shape == (rows, N) and y.dtype == H
    end = int(gl[-1])
    torch.testing.assert_close(y.cpu()[:end].float(), ref[:end].float(), **GMM_TOL)


def test_grouped_matmul_reference_script_shape(ops, dev):
    # benchmark/test_grouped_matmul.py:28-50: 16384 x 2048 -> 768, 128 experts, multinomial routing
    g = _gen(0)
    rows, K, N, E = 16384, 2048, 768, 128
    x = torch.randn(rows, K, generator=g).half()
    w = (0.02 * torch.randn(E, N, K, generator=g)).half().transpose(1, 2)
    sample = torch.multinomial(torch.ones(E), num_samples=rows, replacement=True, generator=g)
    gl = torch.bincount(sample, minlength=E).cumsum(0).to(torch.int64)
    y = ops.grouped_matmul(x.to(dev), w.to(dev), gl.to(dev))
    ref = R.grouped_matmul_ref(x, w, gl)
    torch.testing.assert_close(y.cpu().float(), ref.float(), **GMM_TOL)


def test_grouped_matmul_does_not_write_past_the_last_group(ops, dev):
    x, w, gl = _gmm_case(256, 128, 128, 2, seed=3, counts=[50, 60])
    y = torch.full((256, 128), 5.0, dtype=H, device=dev)
    xd, wd, gd = x.to(dev), w.to(dev), gl.to(dev)
    code = cabi.lib().aops_grouped_matmul_f16(xd.data_ptr(), wd.data_ptr(), gd.data_ptr(), y.data_ptr(), 256, 128, 2, 128,
                                          cabi.stream(dev))
    assert code == 0
    assert torch.all(y[110:] == 5.0)
    ref = R.grouped_matmul_ref(x, w, gl)
    torch.testing.assert_close(y.cpu()[:110].float(), ref[:110].float(), **GMM_TOL)


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7, 8, 9])
@pytest.mark.parametrize(
    "rows,K,N,E,counts",
    [
        (1300, 256, 192, 6, [0, 1, 700, 0, 330, 200]),   # empty groups, one row, 3-tile and 2-tile groups, 69 rows unrouted
        (2500, 384, 576, 300, None),                      # more experts than the per-lane cache of the scan covers
        (4096, 512, 2048, 64, None),                      # several work items per workgroup of the persistent kernel
        (321, 256, 64, 1, [321]),                         # one expert, one row past a full tile, minimum N
    ],
)
def test_grouped_matmul_every_kernel(ops, dev, variant, rows, K, N, E, counts):
    """The tile shape / kernel is normally chosen from the problem size; aops_grouped_matmul_variant_f16 fixes
    one, so that every kernel sees the edge cases (6 = persistent kernel, needs K % 128 == 0, K >= 256; 7, 8 = direct-copy kernels with smaller tiles)."""
    x, w, gl = _gmm_case(rows, K, N, E, seed=variant, counts=counts)
    end = int(gl[-1])
    y = torch.full((rows, N), 5.0, dtype=H, device=dev)
    xd, wd, gd = x.to(dev), w.transpose(1, 2).contiguous().to(dev), gl.to(dev)   # storage [E, N, K]
    code = cabi.lib().aops_grouped_matmul_variant_f16(variant, xd.data_ptr(), wd.data_ptr(), gd.data_ptr(),
                                                      y.data_ptr(), rows, K, E, N, cabi.stream(dev))
    assert code == 0
    ref = R.grouped_matmul_ref(x, w, gl)
    torch.testing.assert_close(y.cpu()[:end].float(), ref[:end].float(), **GMM_TOL)
    assert torch.all(y[end:] == 5.0)


@pytest.mark.parametrize("rows,K,N,E,pad,counts", [
    (1500, 256, 192, 6, 64, None),
    (900, 2048, 320, 3, 64, [0, 650, 250]),       # the row length whose power-of-two stride the padding is for
    (640, 384, 64, 2, 8, [320, 300]),             # the smallest padding; rows past the last group
])
def test_grouped_matmul_with_padded_weight_rows(dev, rows, K, N, E, pad, counts):
    """aops_grouped_matmul_ldw_f16: weight rows ldw = K + pad elements apart.  The padding holds NaN and must never be
    read into a product; the result equals the persistent kernel's on the unpadded weights bit for bit (same kernel,
    same order of operations) and the oracle within tolerance; rows past the last group stay untouched."""
    lib = cabi.lib()
    x, w, gl = _gmm_case(rows, K, N, E, seed=31, counts=counts)
    end = int(gl[-1])
    storage = w.transpose(1, 2).contiguous()                       # [E, N, K]
    padded = torch.full((E, N, K + pad), float("nan"), dtype=H)
    padded[:, :, :K] = storage
    xd, wd, pd, gd = x.to(dev), storage.to(dev), padded.to(dev), gl.to(dev)
    y = torch.full((rows, N), 5.0, dtype=H, device=dev)
    y_ref = torch.full((rows, N), 5.0, dtype=H, device=dev)
    assert lib.aops_grouped_matmul_ldw_f16(xd.data_ptr(), pd.data_ptr(), K + pad, gd.data_ptr(), y.data_ptr(), rows, K, E,
                                           N, cabi.stream(dev)) == 0
    assert lib.aops_grouped_matmul_variant_f16(6, xd.data_ptr(), wd.data_ptr(), gd.data_ptr(), y_ref.data_ptr(), rows, K,
                                               E, N, cabi.stream(dev)) == 0
    assert torch.equal(y, y_ref)
    torch.testing.assert_close(y.cpu()[:end].float(), R.grouped_matmul_ref(x, w, gl)[:end].float(), **GMM_TOL)
    assert torch.all(y[end:] == 5.0)
    # ldw == K is the unpadded operator; a stride below K, or one that breaks the 16-byte alignment of the rows, is refused
    y2 = torch.full((rows, N), 5.0, dtype=H, device=dev)
    assert lib.aops_grouped_matmul_ldw_f16(xd.data_ptr(), wd.data_ptr(), K, gd.data_ptr(), y2.data_ptr(), rows, K, E, N,
                                           cabi.stream(dev)) == 0
    assert torch.equal(y2, y_ref)
    for bad in (K - 8, K + 4):
        assert lib.aops_grouped_matmul_ldw_f16(xd.data_ptr(), pd.data_ptr(), bad, gd.data_ptr(), y.data_ptr(), rows, K, E,
                                               N, cabi.stream(dev)) == -1


def test_measurement_aids_run_and_leave_their_surroundings_alone(dev):
    """The probe entry points (parts of the persistent kernel's k loop switched off; a pure read stream) are
    measurement aids whose results mean nothing, but they must run to completion, refuse what they do not serve, write
    nothing outside y and read nothing outside their operands (guard regions keep their contents)."""
    lib = cabi.lib()
    rows, K, N, E = 700, 256, 192, 5
    x, w, gl = _gmm_case(rows, K, N, E, seed=2, counts=[300, 0, 1, 330, 69])
    xd, wd, gd = x.to(dev), w.transpose(1, 2).contiguous().to(dev), gl.to(dev)
    y = torch.full((rows + 2, N), 7.0, dtype=H, device=dev)        # one guard row on either side
    for parts_off in (9, 11, 13, 6, 14, 1, 8, 25, 27):
        assert lib.aops_grouped_matmul_probe_f16(parts_off, xd.data_ptr(), wd.data_ptr(), K, gd.data_ptr(),
                                                 y[1:].data_ptr(), rows, K, E, N, cabi.stream(dev)) == 0
    torch.cuda.synchronize()
    assert torch.all(y[0] == 7.0) and torch.all(y[-1] == 7.0)
    for bad in (0, 2, 7, 15, -1):
        assert lib.aops_grouped_matmul_probe_f16(bad, xd.data_ptr(), wd.data_ptr(), K, gd.data_ptr(), y[1:].data_ptr(),
                                                 rows, K, E, N, cabi.stream(dev)) == -1
    assert lib.aops_grouped_matmul_probe_f16(9, xd.data_ptr(), wd.data_ptr(), 192, gd.data_ptr(), y[1:].data_ptr(),
                                             rows, 192, E, N, cabi.stream(dev)) == -1    # k the kernel does not take
    assert lib.aops_grouped_matmul_probe_f16(9, xd.data_ptr(), wd.data_ptr(), K - 8, gd.data_ptr(), y[1:].data_ptr(),
                                             rows, K, E, N, cabi.stream(dev)) == -1      # row stride below k
    buf = torch.ones(256 * 1024, dtype=torch.uint8, device=dev)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    for via_lds in (0, 1):
        for seg, row_bytes in ((128, 1024), (256, 512), (512, 512), (1024, 1024), (128, 128)):
            assert lib.aops_probe_read_stream(buf.data_ptr(), buf.numel() // row_bytes, row_bytes, seg, via_lds,
                                              sink.data_ptr(), cabi.stream(dev)) == 0
    torch.cuda.synchronize()
    assert float(sink[0]) == 0.0
    assert lib.aops_probe_read_stream(buf.data_ptr(), 100, 1024, 128, 0, sink.data_ptr(), cabi.stream(dev)) == -1   # rows % 128
    assert lib.aops_probe_read_stream(buf.data_ptr(), 256, 1024, 96, 0, sink.data_ptr(), cabi.stream(dev)) == -1    # piece size
    assert lib.aops_probe_read_stream(buf.data_ptr(), 256, 640, 256, 0, sink.data_ptr(), cabi.stream(dev)) == -1    # not dividing
    assert lib.aops_probe_read_stream(buf.data_ptr(), 256, 1024, 128, 2, sink.data_ptr(), cabi.stream(dev)) == -1   # via_lds
    operands = (torch.rand(16 * 64 * 8, device=dev) - 0.5).half()
    for shape in (16, 32):
        assert lib.aops_probe_mfma_rate(shape, operands.data_ptr(), 64, sink.data_ptr(), cabi.stream(dev)) == 0
    torch.cuda.synchronize()
    assert float(sink[0]) == 0.0
    for shape, iters in ((8, 64), (16, 0), (16, 12), (32, (1 << 20) + 8)):
        assert lib.aops_probe_mfma_rate(shape, operands.data_ptr(), iters, sink.data_ptr(), cabi.stream(dev)) == -1


@pytest.mark.parametrize("seed", range(12))
def test_grouped_matmul_persistent_kernel_random_shapes(ops, dev, seed):
    """The persistent kernel (variant 6) on seeded random problems: group sizes from empty to several tiles (every
    number of live row blocks of a tile occurs), one to many work items per workgroup, 4 to 12 k tiles, so that the
    hand-over of the operand pipeline from one work item to the next is exercised in all its forms."""
    import random
    rnd = random.Random(100 + seed)
    g = _gen(100 + seed)
    E = rnd.choice([1, 3, 8, 33, 70])
    K = 128 * rnd.randint(2, 6)
    N = 64 * rnd.randint(1, 9)
    rows = rnd.choice([31, 321, 700, 1500, 3000])
    routed = rnd.choice([rows, rnd.randint(0, rows)])
    if rnd.random() < 0.5:
        ids = torch.randint(0, E, (routed,), generator=g)
    else:  # skewed: a few large groups, many small or empty ones
        ids = (torch.rand(routed, generator=g) ** 3 * E).long().clamp(0, E - 1)
    gl = torch.bincount(ids, minlength=E).cumsum(0).to(torch.int64)
    x = torch.randn(rows, K, generator=g).half()
    w = (torch.randn(E, K, N, generator=g) / K ** 0.5).half()   # logical [E, K, N]
    y = torch.full((rows, N), 5.0, dtype=H, device=dev)
    xd, wd, gd = x.to(dev), w.transpose(1, 2).contiguous().to(dev), gl.to(dev)   # storage [E, N, K]
    code = cabi.lib().aops_grouped_matmul_variant_f16(6, xd.data_ptr(), wd.data_ptr(), gd.data_ptr(), y.data_ptr(),
                                                      rows, K, E, N, cabi.stream(dev))
    assert code == 0
    ref = R.grouped_matmul_ref(x, w, gl)
    torch.testing.assert_close(y.cpu()[:routed].float(), ref[:routed].float(), **GMM_TOL)
    assert torch.all(y[routed:] == 5.0)


@pytest.mark.parametrize(
    "rows,K,N,E,counts",
    [
        (1300, 256, 192, 6, [0, 1, 700, 0, 330, 200]),   # ragged groups, N/2 = 96 (three column blocks of the last tile)
        (4096, 512, 1536, 64, None),                      # several work items per workgroup
        (700, 2048, 1536, 1, [650]),                      # one expert, rows past the group untouched
        (300, 192, 128, 3, [100, 100, 100]),              # K not a multiple of 128: the small-tile fused kernel
        (90, 256, 192, 20, None),                         # few rows per expert: 64 x 64 tiles, 96 output columns
        (1200, 512, 320, 30, None),                       # 40 rows per expert: 128 x 128 tiles, ragged last column tile
    ],
)
def test_grouped_matmul_swiglu_fused(ops, dev, rows, K, N, E, counts):
    """Fused gate_up + SwiGLU against the oracle chain swiglu_ref(grouped_matmul_ref(...)) with the fp32
    intermediate, and against the unfused device chain."""
    import ascend910a_extras.fused as fused
    x, w, gl = _gmm_case(rows, K, N, E, seed=11, counts=counts)
    end = int(gl[-1])
    xd, wd, gd = x.to(dev), w.to(dev), gl.to(dev)
    y = fused.grouped_matmul_swiglu(xd, wd, gd)
    assert y.shape == (rows, N // 2) and y.dtype == H
    h = torch.zeros(rows, N)
    prev = 0
    for e in range(E):
        t = int(gl[e])
        h[prev:t] = x[prev:t].float() @ w[e].float()
        prev = t
    ref = (torch.nn.functional.silu(h[:, : N // 2]) * h[:, N // 2:]).half()
    torch.testing.assert_close(y.cpu()[:end].float(), ref[:end].float(), **GMM_TOL)
    two = ops.swiglu(ops.grouped_matmul(xd, wd, gd))
    torch.testing.assert_close(y[:end].float(), two[:end].float(), **GMM_TOL)


@pytest.mark.parametrize("m,k,n", [(128, 128, 128), (257, 256, 256), (1, 64, 64), (256, 4096, 1024), (3000, 512, 2048)])
def test_matmul_nt(ops, dev, m, k, n):
    """Legacy dense operator (benchmark/test_matmul.py: x [m,k] @ w[n,k]^T), the grouped matmul without a group_list."""
    g = _gen(m + n)
    x = torch.randn(m, k, generator=g).half()
    w = (torch.randn(n, k, generator=g) / k ** 0.5).half()
    y = ops.matmul(x.to(dev), w.to(dev))
    assert y.shape == (m, n) and y.dtype == H
    torch.testing.assert_close(y.cpu().float(), x.float() @ w.float().T, **GMM_TOL)


SPLIT_K_SHAPES = [(256, 14336, 4096), (16, 8192, 1024), (300, 4096, 256), (1, 2048, 64), (257, 64 * 37, 192),
                  (64, 1024, 2048), (100, 2048, 1024), (512, 16384, 128)]


@pytest.mark.parametrize("m,k,n", SPLIT_K_SHAPES)
def test_matmul_nt_split_k(ops, dev, m, k, n):
    """Few rows and a long k: the k range is split over workgroups and a second kernel adds the partial results.
    Against the fp32 product, against the whole-k kernels, and bit-identical from call to call."""
    g = _gen(m + k + n)
    x = torch.randn(m, k, generator=g).half()
    w = (torch.randn(n, k, generator=g) / k ** 0.5).half()
    xd, wd = x.to(dev), w.to(dev)
    ws_bytes = cabi.lib().aops_matmul_nt_workspace(m, k, n)
    assert ws_bytes > 0, "the shape is meant to take the split-k path"
    y = ops.matmul(xd, wd)
    ref = x.float() @ w.float().T
    torch.testing.assert_close(y.cpu().float(), ref, **GMM_TOL)
    # the whole-k kernel (no workspace) agrees to rounding: both accumulate in fp32, in a different order
    whole = torch.empty_like(y)
    assert cabi.lib().aops_matmul_nt_f16(xd.data_ptr(), wd.data_ptr(), whole.data_ptr(), m, k, n, cabi.stream(dev)) == 0
    torch.testing.assert_close(y.float(), whole.float(), rtol=2e-3, atol=2e-3)
    assert torch.equal(ops.matmul(xd, wd), y)
    # one expert through the grouped entry of the Python API takes the same path
    gl = torch.tensor([m], dtype=torch.int64, device=dev)
    assert torch.equal(ops.grouped_matmul(xd, wd[None].transpose(1, 2), gl), y)
    # a workspace that is too small is refused, the output untouched
    small = torch.empty(ws_bytes - 1, dtype=torch.uint8, device=dev)
    out = torch.zeros_like(y)
    code = cabi.lib().aops_matmul_nt_ws_f16(xd.data_ptr(), wd.data_ptr(), out.data_ptr(), small.data_ptr(), ws_bytes - 1,
                                        m, k, n, cabi.stream(dev))
    torch.cuda.synchronize()
    assert code == -2 and not out.any()


FEW_ROWS_SHAPES = [(1, 4096, 4096), (16, 512, 2048), (7, 576, 2048), (16, 14336, 4096), (9, 4096, 16384),
                   (5, 2112, 2112), (4, 14336, 4096), (3, 2112, 2112), (2, 512, 2048), (4, 6208, 2048)]


@pytest.mark.parametrize("m,k,n", FEW_ROWS_SHAPES)
def test_matmul_nt_few_rows(ops, dev, m, k, n):
    """At most 16 rows (the projections of a small decode batch): one workgroup per 16 rows of W, every wave
    copies its own pieces of W and x into LDS and waits for them alone, no workspace.  Against the fp32 product,
    against the tile kernels, bit-identical from call to call; through the grouped entry the rows past
    group_list[0] stay untouched.  k with a short last piece, n that is not a multiple of the XCD run."""
    g = _gen(m + k + n)
    x = torch.randn(m, k, generator=g).half()
    w = (torch.randn(n, k, generator=g) / k ** 0.5).half()
    xd, wd = x.to(dev), w.to(dev)
    assert cabi.lib().aops_matmul_nt_workspace(m, k, n) == 0
    y = ops.matmul(xd, wd)
    ref = x.float() @ w.float().T
    torch.testing.assert_close(y.cpu().float(), ref, **GMM_TOL)
    assert torch.equal(ops.matmul(xd, wd), y)
    tiles = torch.empty_like(y)                          # the 64 x 64 tile kernel on the same product
    assert cabi.lib().aops_grouped_matmul_variant_f16(5, xd.data_ptr(), wd.data_ptr(), None, tiles.data_ptr(), m, k, 1, n,
                                                      cabi.stream(dev)) == 0
    torch.testing.assert_close(y.float(), tiles.float(), rtol=2e-3, atol=2e-3)
    # one group that ends before the last row: later rows are not written
    part = max(m - 3, 0)
    gl = torch.tensor([part], dtype=torch.int64, device=dev)
    out = torch.full((m, n), 7.0, dtype=H, device=dev)
    code = cabi.lib().aops_grouped_matmul_f16(xd.data_ptr(), wd.data_ptr(), gl.data_ptr(), out.data_ptr(), m, k, 1, n,
                                          cabi.stream(dev))
    torch.cuda.synchronize()
    assert code == 0
    assert torch.equal(out[:part], y[:part]) and bool((out[part:] == 7.0).all())


@pytest.mark.parametrize("m,k,n,part", [(256, 14336, 4096, 200), (64, 4096, 1024, 1), (100, 2048, 512, 0), (128, 8192, 256, 128)])
def test_grouped_matmul_one_expert_split_k_honours_group_list(ops, dev, m, k, n, part):
    """One expert, few rows, long k: the library splits the k range (two kernels, workspace).  Rows at or past
    group_list[0] must stay unwritten there too, as in every other kernel."""
    assert cabi.lib().aops_grouped_matmul_workspace(m, k, 1, n) > 0          # the shape does take the split path
    assert cabi.lib().aops_grouped_matmul_workspace(m, k, 1, n) == cabi.lib().aops_matmul_nt_workspace(m, k, n)
    g = _gen(m + part)
    x = torch.randn(m, k, generator=g).half()
    w = (torch.randn(1, n, k, generator=g) / k ** 0.5).half()
    gl = torch.tensor([part], dtype=torch.int64)
    xd, wd, gd = x.to(dev), w.to(dev), gl.to(dev)
    ws_bytes = cabi.lib().aops_grouped_matmul_workspace(m, k, 1, n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    y = torch.full((m, n), 7.0, dtype=H, device=dev)
    code = cabi.lib().aops_grouped_matmul_ws_f16(xd.data_ptr(), wd.data_ptr(), gd.data_ptr(), y.data_ptr(), ws.data_ptr(),
                                                 ws_bytes, m, k, 1, n, cabi.stream(dev))
    assert code == 0
    torch.cuda.synchronize()
    assert bool((y[part:] == 7.0).all())
    ref = x.float() @ w[0].float().T
    torch.testing.assert_close(y[:part].cpu().float(), ref[:part], **GMM_TOL)
    # the Python API takes the same path; its fresh output holds the same rows
    y_api = ops.grouped_matmul(xd, wd.transpose(1, 2), gd)
    assert torch.equal(y_api[:part], y[:part])
    # a workspace that is wanted but too small is refused
    assert cabi.lib().aops_grouped_matmul_ws_f16(xd.data_ptr(), wd.data_ptr(), gd.data_ptr(), y.data_ptr(), ws.data_ptr(),
                                                 ws_bytes - 1, m, k, 1, n, cabi.stream(dev)) == -2


def test_matmul_nt_ws_without_split(ops, dev):
    """Shapes with enough output tiles need no workspace; the workspace entry point then equals the plain one."""
    m, k, n = 512, 512, 8192
    assert cabi.lib().aops_matmul_nt_workspace(m, k, n) == 0
    g = _gen(5)
    x = torch.randn(m, k, generator=g).half().to(dev)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).half().to(dev)
    a, b = torch.empty(m, n, dtype=H, device=dev), torch.empty(m, n, dtype=H, device=dev)
    assert cabi.lib().aops_matmul_nt_ws_f16(x.data_ptr(), w.data_ptr(), a.data_ptr(), None, 0, m, k, n, cabi.stream(dev)) == 0
    assert cabi.lib().aops_matmul_nt_f16(x.data_ptr(), w.data_ptr(), b.data_ptr(), m, k, n, cabi.stream(dev)) == 0
    assert torch.equal(a, b)


def test_persistent_kernel_with_256_row_tiles(ops, dev):
    """8192 rows in one group and 2048 columns: 256-row tiles cover the rows in 32 work items per column tile where
    320-row tiles would need 26 with the last one mostly empty, so the library takes the 256-row form of the
    persistent kernel - plain, with the fused activation, and with the row gather."""
    import ascend910a_extras.ascend910a_extras_C as C
    import ascend910a_extras.fused as fused
    g = _gen(41)
    rows, K, N = 8192, 256, 2048
    x = torch.randn(rows, K, generator=g).half()
    w = (torch.randn(1, N, K, generator=g) / K ** 0.5).half().transpose(1, 2)
    gl = torch.tensor([rows - 100], dtype=torch.int64)
    xd, wd, gd = x.to(dev), w.to(dev), gl.to(dev)
    end = int(gl[-1])
    ref = x.float() @ w[0].float()
    y = ops.grouped_matmul(xd, wd, gd)
    torch.testing.assert_close(y[:end].cpu().float(), ref[:end], **GMM_TOL)
    act = fused.grouped_matmul_swiglu(xd, wd, gd)
    act_ref = (torch.nn.functional.silu(ref[:, : N // 2]) * ref[:, N // 2:])
    torch.testing.assert_close(act[:end].cpu().float(), act_ref[:end], **GMM_TOL)
    perm = torch.randperm(rows, generator=g).int()
    gathered = C.grouped_matmul_swiglu_gather(xd, perm.to(dev), 1, wd, gd)
    assert torch.equal(gathered[:end], fused.grouped_matmul_swiglu(xd[perm.long().to(dev)], wd, gd)[:end])


def test_dense_mlp_chain(ops, dev):
    """benchmark/test_mlp.py:37-41 through grouped_matmul with one expert (reduced width)."""
    g = _gen(0)
    bs, hidden, inter = 256, 1024, 3584
    x = torch.randn(bs, hidden, generator=g).half()
    gu = (0.02 * torch.randn(2 * inter, hidden, generator=g)).half()
    dn = (0.02 * torch.randn(hidden, inter, generator=g)).half()
    gl = torch.tensor([bs], dtype=torch.int64).to(dev)
    h = ops.grouped_matmul(x.to(dev), gu.to(dev)[None].transpose(1, 2), gl)
    h = ops.swiglu(h)
    y = ops.grouped_matmul(h, dn.to(dev)[None].transpose(1, 2), gl)
    torch.testing.assert_close(y.cpu().float(), R.mlp_ref(x, gu, dn).float(), **GMM_TOL)


@pytest.mark.parametrize("pattern", ["prefill", "random", "mixed"])
@pytest.mark.parametrize("with_value", [True, False])
def test_reshape_and_cache_prefill_sized(ops, dev, pattern, with_value):
    """Prefill-sized calls, bit-exact for the slot patterns a caller produces: whole pages in token order, a random
    permutation, and a mix with a swapped pair, slots outside the cache, a run that crosses a page boundary and a
    token count that is not a multiple of anything."""
    g = _gen(31)
    Hkv, D, NB, P = 8, 128, 96, 128
    T = 4096 + (0 if pattern == "prefill" else 13)
    assert (T + P - 1) // P <= NB // 2
    key = torch.randn(T, Hkv, D, generator=g).half()
    value = torch.randn(T, Hkv, D, generator=g).half()
    if pattern == "random":
        slots = torch.randperm(NB * P, generator=g)[:T].int()
    else:
        pages = 2 * torch.randperm(NB // 2, generator=g)[: (T + P - 1) // P]   # even pages: the odd ones stay free
        slots = (pages[:, None] * P + torch.arange(P)[None, :]).reshape(-1)[:T].int()
        if pattern == "mixed":
            slots[40], slots[41] = slots[41].clone(), slots[40].clone()   # run broken inside a tile
            slots[100] = -1                                                 # skipped token
            slots[200] = NB * P                                             # outside the cache
            slots[352:384] = slots[352:384] + 16                            # consecutive, but crossing into the next page
    kc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()
    vc0 = torch.randn(NB, Hkv * D // 16, P, 16, generator=g).half()
    kcd, vcd = kc0.to(dev), vc0.to(dev)
    kc_ref, vc_ref = kc0.clone(), vc0.clone()
    if pattern == "mixed":  # duplicate targets would make the result depend on the write order: keep slots unique
        valid = slots[(slots >= 0) & (slots < NB * P)]
        assert valid.unique().numel() == valid.numel()
    if with_value:
        ops.reshape_and_cache(key.to(dev), value.to(dev), kcd, vcd, slots.to(dev))
        R.reshape_and_cache_ref(key, kc_ref, slots, value, vc_ref)
    else:
        ops.reshape_and_cache(key.to(dev), None, kcd, None, slots.to(dev))
        R.reshape_and_cache_ref(key, kc_ref, slots)
    assert torch.equal(kcd.cpu(), kc_ref)
    assert torch.equal(vcd.cpu(), vc_ref)


# ----------------------------------------------------------------------------- paged attention
def _paged_case(B, Hq, Hkv, D, P, lens, seed, max_pages=None, extra_pages=5, poison=False):
    g = _gen(seed)
    pages_per = [(l + P - 1) // P for l in lens]
    max_pages = max_pages or max(max(pages_per), 1)
    NB = sum(pages_per) + extra_pages
    perm = torch.randperm(NB, generator=g)
    bt = torch.full((B, max_pages), -1 if poison else 0, dtype=torch.int32)
    c = 0
    used = torch.zeros(NB, P, dtype=torch.bool)
    for b, n in enumerate(pages_per):
        bt[b, :n] = perm[c:c + n].int()
        for j in range(lens[b]):
            used[int(bt[b, j // P]), j % P] = True
        c += n
    kd = torch.randn(NB, P, Hkv, D, generator=g).half()
    vd = torch.randn(NB, P, Hkv, D, generator=g).half()
    if poison:
        kd[~used] = float("nan")
        vd[~used] = float("nan")
    q = torch.randn(B, Hq, D, generator=g).half()
    return q, R.nz_pack(kd), R.nz_pack(vd), bt, torch.tensor(lens, dtype=torch.int32)


def _run_pa(ops, dev, case):
    q, kc, vc, bt, cl = case
    return ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), bt.to(dev), cl.to(dev)).cpu()


@pytest.mark.parametrize(
    "B,Hq,Hkv,P,lens",
    [
        (4, 32, 8, 128, [512, 4096, 1000, 37]),
        (6, 32, 8, 128, [1, 2, 31, 32, 33, 129]),
        (3, 8, 8, 32, [100, 1, 700]),          # no GQA, small pages
        (2, 16, 8, 64, [64, 65]),               # group of 2
        (2, 16, 2, 128, [300, 2049]),           # group of 8
        (3, 32, 8, 128, [0, 128, 0]),           # empty sequences
    ],
)
def test_paged_attention(ops, dev, B, Hq, Hkv, P, lens):
    case = _paged_case(B, Hq, Hkv, 128, P, lens, seed=0)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    assert o.shape == (B, Hq, 128) and o.dtype == H
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    # the op's error is far below the bar: typical |o| ~ 0.05, so also check a tight absolute error
    assert (o.float() - ref.float()).abs().max() < 2e-3


@pytest.mark.parametrize("D,P,Hq,Hkv", [(128, 128, 32, 8), (64, 16, 6, 2)])
def test_paged_attention_clamps_block_table_entries(ops, dev, D, P, Hq, Hkv):
    """Block-table entries outside the cache are clamped into it (both kernels): the sequences with valid tables are
    unaffected, the sequence with bad entries equals the result for the clamped table."""
    lens = [3 * P + 5, 2 * P, P + 1]
    q, kc, vc, bt, cl = _paged_case(3, Hq, Hkv, D, P, lens, seed=4)
    NB = kc.size(0)
    bad = bt.clone()
    bad[1, 0] = NB + 1000
    bad[1, 1] = -7
    o = ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), bad.to(dev), cl.to(dev)).cpu()
    clamped = bad.clone().clamp_(0, NB - 1)
    ref = R.paged_attention_ref(q, kc, vc, clamped, cl)
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    good = R.paged_attention_ref(q, kc, vc, bt, cl)
    torch.testing.assert_close(o[[0, 2]].float(), good[[0, 2]].float(), **TOL)


@pytest.mark.parametrize("B,Hq,Hkv,P", [(150, 8, 2, 64), (70, 4, 1, 128), (1030, 2, 1, 32)])
def test_paged_attention_batch_larger_than_a_wave(ops, dev, B, Hq, Hkv, P):
    """More than 64 sequences: a one-workgroup kernel ranks the sequences by length (up to 1024 of them; beyond that
    they are taken in index order) and the workgroups take them longest first; with few kv heads the sequences are
    also cut into several chunks.  Ties, empty sequences and one very long sequence included."""
    rnd = torch.Generator().manual_seed(12)
    lens = torch.randint(0, 600, (B,), generator=rnd).tolist()
    lens[3] = 0
    lens[5] = lens[6] = lens[60] = 333
    lens[B // 2] = 2500
    case = _paged_case(B, Hq, Hkv, 128, P, lens, seed=12)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    assert (o.float() - ref.float()).abs().max() < 3e-3


@pytest.mark.parametrize(
    "B,Hq,Hkv,D,P,lens",
    [
        (3, 8, 2, 64, 16, [1, 50, 200]),        # head_dim 64, small pages
        (2, 6, 2, 128, 128, [130, 700]),        # 3 query heads per kv head
        (2, 4, 4, 256, 32, [33, 0]),            # head_dim 256, one empty sequence
        (2, 32, 2, 128, 64, [100, 1000]),       # 16 query heads per kv head (matrix-core path)
        (2, 8, 2, 128, 24, [25, 300]),          # block size not a multiple of 16: generic kernel
        (1, 5, 5, 48, 8, [77]),                 # head_dim 48 on 8-token pages: generic kernel
        (2, 32, 1, 64, 16, [70, 300]),          # more than 16 query heads per kv head
        (2, 24, 1, 64, 32, [33, 129]),
        (3, 17, 1, 64, 16, [1, 16, 250]),
        (2, 40, 2, 128, 16, [100, 37]),         # 20 heads per kv head at head_dim 128
    ],
)
def test_paged_attention_other_shapes(ops, dev, B, Hq, Hkv, D, P, lens):
    case = _paged_case(B, Hq, Hkv, D, P, lens, seed=3, poison=True)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    assert o.shape == (B, Hq, D)
    assert not torch.isnan(o).any()
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    assert (o.float() - ref.float()).abs().max() < 3e-3


@pytest.mark.parametrize(
    "B,Hq,Hkv,P,lens",
    [
        (3, 24, 8, 128, [130, 700, 2500]),      # 3 query heads per kv head
        (2, 10, 2, 64, [64, 1000]),             # 5
        (2, 12, 2, 128, [1, 300]),              # 6
        (2, 14, 2, 32, [31, 33]),               # 7
        (2, 24, 2, 128, [257, 4000]),           # 12
        (4, 32, 8, 16, [16, 17, 300, 1]),       # 16-token pages: the two halves of a step lie in different pages
        (3, 32, 8, 48, [48, 96, 1000]),         # page size an odd multiple of 16; lengths that fill the last page
        (2, 6, 2, 80, [79, 2000]),              # 3 heads per kv head on 80-token pages
        (2, 16, 4, 144, [144, 145]),
    ],
)
def test_paged_attention_matrix_core_path_any_group_and_page_size(ops, dev, B, Hq, Hkv, P, lens):
    """head_dim 128 takes the matrix-core kernel for every group size up to 16 and every page size that is a multiple
    of 16; unused cache slots hold NaN and unused table entries -1."""
    assert cabi.lib().aops_paged_attention_workspace(B, Hq, Hkv, 128, P, 64) > 16   # not the generic kernel
    case = _paged_case(B, Hq, Hkv, 128, P, lens, seed=9, poison=True)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    assert not torch.isnan(o).any()
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    assert (o.float() - ref.float()).abs().max() < 3e-3


@pytest.mark.parametrize(
    "B,Hq,Hkv,D,P,lens",
    [
        (4, 32, 8, 64, 128, [512, 4096, 1000, 37]),     # head_dim 64, sequences split into chunks
        (3, 16, 2, 64, 16, [1, 50, 2000]),              # 8 heads per kv head on 16-token pages
        (2, 12, 4, 64, 48, [48, 300]),
        (3, 16, 8, 256, 128, [130, 3000, 1]),           # head_dim 256
        (2, 16, 2, 256, 32, [33, 700]),                 # 8 heads per kv head: the largest group at 256
        (2, 3, 1, 256, 64, [64, 65]),
    ],
)
def test_paged_attention_matrix_core_path_other_head_sizes(ops, dev, B, Hq, Hkv, D, P, lens):
    assert cabi.lib().aops_paged_attention_workspace(B, Hq, Hkv, D, P, 64) > 16   # not the generic kernel
    case = _paged_case(B, Hq, Hkv, D, P, lens, seed=13, poison=True)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    assert o.shape == (B, Hq, D) and not torch.isnan(o).any()
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    assert (o.float() - ref.float()).abs().max() < 3e-3


@pytest.mark.parametrize(
    "B,Hq,Hkv,P,maxlen,seed",
    [
        (40, 32, 8, 128, 3000, 1),     # 320 (sequence, kv head) pairs: more units than shares, several sequences per share
        (63, 8, 2, 64, 1200, 2),       # 128 shares per kv head
        (5, 4, 1, 128, 9000, 3),       # 256 shares for five sequences: long sequences cut into many partial results
        (33, 16, 4, 16, 700, 4),       # 16-token pages
        (12, 32, 8, 128, 255, 5),      # every sequence shorter than one 256-token unit
        (64, 32, 8, 128, 9000, 6),     # 512 pairs, but a block table wide enough for one long sequence among short ones
        (130, 32, 8, 128, 9000, 7),    # more than 64 sequences: the partition comes from a one-workgroup plan kernel
        (1100, 2, 1, 64, 4500, 8),     # more sequences than the plan kernel has threads
    ],
)
def test_paged_attention_balanced_partition(ops, dev, B, Hq, Hkv, P, maxlen, seed):
    """Batches with fewer than two (sequence, kv head) pairs per CU, or whose block table allows contexts beyond 4096
    tokens: the token stream is cut into equal shares of 256-token units, one per workgroup, whatever the sequence
    boundaries; a share may hold the end of one sequence, whole sequences and the start of another.  Empty sequences
    in between, NaN in unused slots.  Up to 64 sequences every wave derives the partition itself; above that a
    one-workgroup kernel writes it into the workspace first."""
    import random
    rnd = random.Random(seed)
    lens = [rnd.choice([0, 1, 255, 256, 257, rnd.randint(1, maxlen), rnd.randint(1, maxlen)]) for _ in range(B)]
    lens[rnd.randrange(B)] = maxlen
    case = _paged_case(B, Hq, Hkv, 128, P, lens, seed=seed, poison=True)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    assert not torch.isnan(o).any()
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    assert (o.float() - ref.float()).abs().max() < 3e-3
    # deterministic: the partial results are merged in a fixed order
    assert torch.equal(_run_pa(ops, dev, case), o)


def test_paged_attention_only_odd_page_sizes_take_the_generic_kernel():
    """Every head size and every number of query heads per kv head runs on the matrix cores as long as the page size
    is a multiple of 16 tokens; the generic kernel, which needs no workspace (the query answers 16), is left with the
    other page sizes."""
    ws = cabi.lib().aops_paged_attention_workspace
    for hq, hkv, d in [(32, 1, 64), (24, 1, 64), (17, 1, 64), (40, 2, 128), (9, 1, 256), (80, 1, 128), (4, 4, 48),
                       (16, 4, 96), (8, 2, 160), (8, 8, 16), (6, 2, 240)]:
        assert ws(2, hq, hkv, d, 16, 64) > 16
    for p in (8, 24, 100):
        assert ws(2, 32, 8, 128, p, 64) == 16


@pytest.mark.parametrize("D", [16, 32, 48, 80, 96, 112, 144, 160, 176, 192, 208, 224, 240])
@pytest.mark.parametrize(
    "B,Hq,Hkv,P,lens",
    [
        (3, 8, 2, 16, [1, 50, 700]),            # whole sequences per workgroup or few chunks
        (2, 6, 2, 128, [3000, 257]),            # balanced partition, sequences cut into partial results
        (70, 4, 4, 32, None),                   # more sequences than lanes
    ],
)
def test_paged_attention_every_head_size(ops, dev, D, B, Hq, Hkv, P, lens):
    """Head sizes that are a multiple of 16 but not 64, 128 or 256: whole slices of 32 elements plus, for odd multiples
    of 16, a half slice whose upper lanes hold zeros.  Unused cache slots hold NaN and unused table entries -1."""
    if lens is None:
        rnd = torch.Generator().manual_seed(D)
        lens = torch.randint(0, 400, (B,), generator=rnd).tolist()
        lens[7] = 1500
    assert cabi.lib().aops_paged_attention_workspace(B, Hq, Hkv, D, P, 64) > 16   # not the generic kernel
    case = _paged_case(B, Hq, Hkv, D, P, lens, seed=D + B, poison=True)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    assert o.shape == (B, Hq, D) and not torch.isnan(o).any()
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    assert (o.float() - ref.float()).abs().max() < 3e-3


@pytest.mark.parametrize(
    "B,Hq,Hkv,D,P,lens",
    [
        (2, 17, 1, 64, 16, [1, 250]),           # 17 heads per kv head: two sub-groups, the second with one head
        (2, 24, 1, 128, 32, [33, 1290]),        # 24
        (3, 64, 2, 128, 128, [130, 5000, 0]),   # 32: two full sub-groups per workgroup; balanced partition
        (2, 40, 1, 64, 16, [70, 300]),          # 40: two workgroups per kv head (32 + 8 heads)
        (2, 80, 2, 96, 48, [100, 1000]),        # 40 at head_dim 96
        (2, 20, 1, 256, 64, [64, 65]),          # above head_dim 128 a workgroup serves 16 heads: 16 + 4
        (2, 36, 2, 192, 16, [700, 3]),          # 18 at head_dim 192
        (2, 16, 1, 256, 32, [33, 700]),         # 16 heads at head_dim 256: the cross-wave merge runs in passes
        (70, 48, 2, 128, 16, None),             # 24 heads per kv head, more sequences than lanes
    ],
)
def test_paged_attention_wide_groups(ops, dev, B, Hq, Hkv, D, P, lens):
    """More than 16 query heads per kv head: a workgroup serves up to two sub-groups of 16 heads from one set of K/V
    registers (head_dim up to 128), and kv heads with more query heads than that are shared by several workgroups."""
    if lens is None:
        rnd = torch.Generator().manual_seed(5)
        lens = torch.randint(0, 300, (B,), generator=rnd).tolist()
        lens[11] = 2000
    assert cabi.lib().aops_paged_attention_workspace(B, Hq, Hkv, D, P, 128) > 16
    case = _paged_case(B, Hq, Hkv, D, P, lens, seed=17, poison=True)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    assert o.shape == (B, Hq, D) and not torch.isnan(o).any()
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    assert (o.float() - ref.float()).abs().max() < 3e-3
    assert torch.equal(_run_pa(ops, dev, case), o)


def test_paged_attention_very_long_context(ops, dev):
    """Contexts of 200000 and 70000 tokens next to one of 5: 782 units of 256 tokens cut into 128 shares per kv
    head, more than 100 partial results for the longest sequence."""
    case = _paged_case(3, 8, 2, 128, 128, [200000, 70000, 5], seed=21)
    o = _run_pa(ops, dev, case)
    ref = R.paged_attention_ref(*case)
    torch.testing.assert_close(o.float(), ref.float(), **TOL)
    assert (o.float() - ref.float()).abs().max() < 3e-3


def test_paged_attention_ignores_garbage_and_unused_table_entries(ops, dev):
    lens = [5, 130, 257, 1]
    clean = _paged_case(4, 32, 8, 128, 128, lens, seed=1, max_pages=6)
    dirty = _paged_case(4, 32, 8, 128, 128, lens, seed=1, max_pages=6, poison=True)
    o_clean = _run_pa(ops, dev, clean)
    o_dirty = _run_pa(ops, dev, dirty)
    assert not torch.isnan(o_dirty).any()
    assert torch.equal(o_clean, o_dirty)


def test_paged_attention_special_cases(ops, dev):
    q, kc, vc, bt, cl = _paged_case(3, 32, 8, 128, 128, [1, 640, 200], seed=2)
    o = _run_pa(ops, dev, (q, kc, vc, bt, cl))
    # L = 1 -> o = V_0 exactly (softmax weight 1)
    v0 = R.gather_kv_from_cache(vc, bt[0], 1, 8)[0]
    for h in range(32):
        assert torch.equal(o[0, h], v0[h // 4])
    # identical queries inside a GQA group give identical outputs
    q2 = q.clone(); q2[:, 1] = q2[:, 0]
    o2 = _run_pa(ops, dev, (q2, kc, vc, bt, cl))
    assert torch.equal(o2[:, 0], o2[:, 1])
    # permuting physical pages together with the table changes nothing (bitwise)
    NB = kc.shape[0]
    perm = torch.randperm(NB, generator=_gen(5))
    inv = torch.empty_like(perm); inv[perm] = torch.arange(NB)
    o3 = _run_pa(ops, dev, (q, kc[perm], vc[perm], inv[bt.long()].int(), cl))
    assert torch.equal(o3, o)
    # large scores: keys aligned with the query must not overflow the softmax
    q4 = (q * 6).half()
    kd = R.nz_unpack(kc, 8); j = 77
    kd[int(bt[1, 0]), j] = q4[1, ::4] * 1.0
    o4 = _run_pa(ops, dev, (q4, R.nz_pack(kd), vc, bt, cl))
    ref4 = R.paged_attention_ref(q4, R.nz_pack(kd), vc, bt, cl)
    assert torch.isfinite(o4).all()
    torch.testing.assert_close(o4.float(), ref4.float(), **TOL)


def test_decode_step_pipeline(ops, dev):
    """rope -> reshape_and_cache of the new token at position ctx-1 -> paged attention, in the
    order of the reference's decoder layer (csrc/ffi/graph.cpp:255-358)."""
    g = _gen(0)
    B, Hq, Hkv, D, P = 8, 32, 8, 128, 128
    lens = torch.randint(1, 1500, (B,), generator=g).tolist()
    q, kc, vc, bt, cl = _paged_case(B, Hq, Hkv, D, P, lens, seed=4)
    k_new = torch.randn(B, Hkv, D, generator=g).half()
    v_new = torch.randn(B, Hkv, D, generator=g).half()
    cos, sin = R.build_cos_sin_cache(4096, D, theta=1e6)
    pos = (cl - 1).int()
    slots = torch.tensor([int(bt[b, int(pos[b]) // P]) * P + int(pos[b]) % P for b in range(B)], dtype=torch.int32)
    # oracle
    rq, rk = R.rope_ref(q, k_new, pos, cos, sin)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    R.reshape_and_cache_ref(rk, kc_ref, slots, v_new, vc_ref)
    o_ref = R.paged_attention_ref(rq, kc_ref, vc_ref, bt, cl)
    # device
    kcd, vcd = kc.to(dev), vc.to(dev)
    oq, ok = ops.rope(q.to(dev), k_new.to(dev), pos.to(dev), cos.to(dev), sin.to(dev))
    ops.reshape_and_cache(ok, v_new.to(dev), kcd, vcd, slots.to(dev))
    o = ops.paged_attention(oq, kcd, vcd, bt.to(dev), cl.to(dev))
    assert torch.equal(vcd.cpu(), vc_ref)
    torch.testing.assert_close(o.cpu().float(), o_ref.float(), **TOL)


def test_ops_run_on_the_current_stream(ops, dev):
    """The launchers enqueue on torch's current stream (reference: getCurrentNPUStream)."""
    x = torch.randn(64, 256, device=dev, dtype=H)
    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(s):
        y = ops.swiglu(x)
    s.synchronize()
    torch.testing.assert_close(y.cpu().float(), R.swiglu_ref(x.cpu()).float(), **TOL)


def test_print_info(ops, dev, capsys):
    ops.print_info()
    out = capsys.readouterr().out
    assert "compute units" in out and "gfx" in out


def test_caches_larger_than_4_gib(ops, dev):
    """Page offsets beyond 2^32 bytes (and 2^31 elements): reshape_and_cache, the fused rope + cache write and paged
    attention on 5.4 GB caches whose pages in use lie at the far end.  Only those pages are ever initialised or
    copied to the host; the oracle works on a compact copy with a remapped block table."""
    import ascend910a_extras.fused as fused

    g = _gen(77)
    NB, Hkv, Hq, D, P = 20480, 8, 32, 128, 128
    assert NB * (Hkv * D // 16) * P * 16 > 2 ** 31
    kc = torch.empty(NB, Hkv * D // 16, P, 16, dtype=H, device=dev)
    vc = torch.empty_like(kc)
    B, lens = 3, [300, 128, 1]
    used = [NB - 1, NB - 7, 16400, NB - 300, 17000]                 # pages beyond element 2^31, not in order
    bt = torch.tensor([[used[0], used[1], used[2]], [used[3], 0, 0], [used[4], 0, 0]], dtype=torch.int32)
    small_k = torch.randn(len(used), Hkv * D // 16, P, 16, generator=g).half()
    small_v = torch.randn(len(used), Hkv * D // 16, P, 16, generator=g).half()
    idx = torch.tensor(used, device=dev)
    kc[idx] = small_k.to(dev)
    vc[idx] = small_v.to(dev)
    remap = {p: i for i, p in enumerate(used)}
    bt_small = torch.tensor([[remap.get(int(p), 0) for p in row] for row in bt], dtype=torch.int32)
    cl = torch.tensor(lens, dtype=torch.int32)
    # the newest token of every sequence arrives through rope + cache write
    q = torch.randn(B, Hq, D, generator=g).half()
    k = torch.randn(B, Hkv, D, generator=g).half()
    v = torch.randn(B, Hkv, D, generator=g).half()
    pos = (cl - 1).int()
    cos, sin = R.build_cos_sin_cache(512, D)
    slots = torch.tensor([int(bt[b, int(pos[b]) // P]) * P + int(pos[b]) % P for b in range(B)], dtype=torch.int32)
    slots_small = torch.tensor([int(bt_small[b, int(pos[b]) // P]) * P + int(pos[b]) % P for b in range(B)], dtype=torch.int32)
    assert int(slots.max()) * (Hkv * D) > 2 ** 31
    oq = fused.rope_reshape_and_cache(q.to(dev), k.to(dev), v.to(dev), pos.to(dev), cos.to(dev), sin.to(dev), kc, vc,
                                      slots.to(dev))
    rq, rk = R.rope_ref(q, k, pos, cos, sin)
    R.reshape_and_cache_ref(rk, small_k, slots_small, v, small_v)
    assert torch.equal(kc[idx].cpu(), small_k) and torch.equal(vc[idx].cpu(), small_v)
    # the plain operator writes the same bytes
    kc2 = torch.empty_like(kc)
    ops.reshape_and_cache(rk.to(dev), None, kc2, None, slots.to(dev))
    for b in range(B):
        page, off = int(slots[b]) // P, int(slots[b]) % P
        assert torch.equal(kc2[page, :, off, :].cpu(), small_k[remap[page], :, off, :])
    del kc2
    o = ops.paged_attention(oq, kc, vc, bt.to(dev), cl.to(dev)).cpu()
    ref = R.paged_attention_ref(rq, small_k, small_v, bt_small, cl)
    torch.testing.assert_close(o.float(), ref.float(), **TOL)


def test_grouped_matmul_more_than_2_31_elements(ops, dev):
    """Row offsets beyond 2^31 elements of x (4.9 GB of activations): slices at the start, across a group boundary far
    into the matrix and at the very end against the fp32 product of the same rows."""
    rows, K, N, E = 1_200_000, 2048, 64, 3
    assert rows * K > 2 ** 31
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.empty(rows, K, dtype=H, device=dev)
    for r0 in range(0, rows, 100_000):
        x[r0:r0 + 100_000] = torch.randn(min(100_000, rows - r0), K, generator=g, device=dev).half()
    w = (torch.randn(E, N, K, generator=g, device=dev) / K ** 0.5).half().transpose(1, 2)
    bounds = [400_000, 800_037, rows]
    gl = torch.tensor(bounds, dtype=torch.int64, device=dev)
    y = ops.grouped_matmul(x, w, gl)
    for lo, hi in ((0, 512), (800_037 - 300, 800_037 + 300), (rows - 512, rows)):
        xs = x[lo:hi].float().cpu()
        ref = torch.empty(hi - lo, N)
        for r in range(lo, hi):
            e = sum(r >= b for b in bounds)
            ref[r - lo] = xs[r - lo] @ w[e].float().cpu()
        torch.testing.assert_close(y[lo:hi].cpu().float(), ref, **GMM_TOL)
