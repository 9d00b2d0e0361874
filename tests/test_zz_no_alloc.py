"""The paged-attention entry point that allocates nothing (`aops_paged_attention_noalloc_f16`, for callers that
cannot call hipMalloc: code under HIP graph capture, tight serving loops) against the existing entry point with a
caller's workspace, through the C ABI.  Both run the same kernels, so the outputs must agree bit for bit; each
case makes two calls in a row on the shared static scratch, the second on a smaller input, so that stale
contents of the first call would show."""
import pytest
import torch

import cabi
import oracle.ops_ref as R

pytestmark = pytest.mark.gpu
H = torch.float16


def _case(B, Hq, Hkv, D, P, lens, seed, max_pages):
    g = torch.Generator().manual_seed(seed)
    pages_per = [(l + P - 1) // P for l in lens]
    NB = sum(pages_per) + 3
    perm = torch.randperm(NB, generator=g)
    bt = torch.zeros(B, max_pages, dtype=torch.int32)
    c = 0
    for b, n in enumerate(pages_per):
        bt[b, :n] = perm[c:c + n].int()
        c += n
    kd = torch.randn(NB, P, Hkv, D, generator=g).half()
    vd = torch.randn(NB, P, Hkv, D, generator=g).half()
    q = torch.randn(B, Hq, D, generator=g).half()
    return q, R.nz_pack(kd), R.nz_pack(vd), bt, torch.tensor(lens, dtype=torch.int32)


def _both(dev, case, Hkv):
    """(output of the workspace entry point, output of the no-allocation entry point), same inputs."""
    lib = cabi.lib()
    q, kc, vc, bt, cl = (t.to(dev) for t in case)
    B, Hq, D = q.shape
    NB, _, P, _ = kc.shape
    max_pages = bt.size(1)
    ws_bytes = lib.aops_paged_attention_workspace(B, Hq, Hkv, D, P, max_pages)
    assert 0 < ws_bytes <= 32 * 1024 * 1024
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    want = torch.full_like(q, float("nan"))
    got = torch.full_like(q, float("nan"))
    s = cabi.stream(dev)
    assert lib.aops_paged_attention_f16(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(), cl.data_ptr(),
                                        want.data_ptr(), ws.data_ptr(), ws_bytes, B, Hq, Hkv, D, P, max_pages, NB, s) == 0
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    reserved_before = torch.cuda.memory_reserved(dev)
    assert lib.aops_paged_attention_noalloc_f16(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(),
                                                cl.data_ptr(), got.data_ptr(), B, Hq, Hkv, D, P, max_pages, NB, s) == 0
    torch.cuda.synchronize()
    # no device memory was taken by the call (another process on the GPU may free memory meanwhile, so the free
    # amount may grow; torch's own pool must not have moved at all)
    assert torch.cuda.mem_get_info()[0] >= free_before
    assert torch.cuda.memory_reserved(dev) == reserved_before
    return want.cpu(), got.cpu(), ws_bytes


# (first call, second smaller call): shapes that take the balanced partition + merge (few sequences), fixed
# chunks + merge, the partition of more than 64 sequences (wide block table), whole sequences per workgroup (no
# partial results), small pages, the generic kernel (no scratch at all), head_dim 256 and a head size with a half
# slice, more than 16 query heads per kv head, and more than 64 sequences with a narrow table (length ranking in
# the int area behind few partial results)
PAIRS = [
    ((8, 32, 8, 128, 128, [4000, 700, 130, 2900, 3300, 512, 1, 2048], 32), (3, 32, 8, 128, 128, [300, 1500, 64], 32)),
    ((1, 32, 8, 128, 128, [20000], 160), (1, 32, 8, 128, 128, [3000], 24)),
    ((70, 8, 2, 128, 64, None, 128), (66, 8, 2, 128, 64, None, 70)),
    ((64, 32, 8, 128, 128, None, 32), (64, 32, 8, 128, 128, None, 8)),
    ((4, 6, 2, 64, 16, [1000, 17, 640, 2000], 128), (2, 6, 2, 64, 16, [33, 200], 16)),
    ((2, 5, 5, 48, 8, [77, 300], 40), (1, 5, 5, 48, 8, [9], 2)),
    ((6, 16, 2, 256, 64, [3000, 64, 700, 1, 4096, 129], 64), (2, 16, 2, 256, 64, [500, 65], 8)),
    ((5, 12, 4, 80, 32, [2500, 31, 900, 33, 1], 80), (3, 12, 4, 80, 32, [100, 300, 7], 10)),
    ((3, 48, 2, 128, 16, [1800, 40, 600], 120), (2, 48, 2, 128, 16, [90, 16], 6)),
    ((200, 8, 2, 128, 32, None, 4), (80, 8, 2, 128, 32, None, 2)),
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_noalloc_entry_equals_workspace_entry_twice_in_a_row(dev, first, second):
    for idx, (B, Hq, Hkv, D, P, lens, max_pages) in enumerate((first, second)):
        if lens is None:
            g = torch.Generator().manual_seed(B + max_pages)
            lens = torch.randint(1, max_pages * P + 1, (B,), generator=g).tolist()
        case = _case(B, Hq, Hkv, D, P, lens, seed=7 + idx, max_pages=max_pages)
        want, got, _ = _both(dev, case, Hkv)
        assert not torch.isnan(want).any()
        assert torch.equal(got, want), f"call {idx}: the two entry points disagree"
        if idx == 1:   # the smaller second call also against the oracle
            ref = R.paged_attention_ref(*case)
            torch.testing.assert_close(got.float(), ref.float(), rtol=1e-2, atol=1e-2)


def test_noalloc_entry_refuses_what_its_scratch_cannot_hold(dev):
    lib = cabi.lib()
    # 64 sequences with a block table that allows 32768 tokens: 34 MB of partial results
    assert lib.aops_paged_attention_workspace(64, 32, 8, 128, 128, 256) > 32 * 1024 * 1024
    z = torch.zeros(16, dtype=H, device=dev)
    code = lib.aops_paged_attention_noalloc_f16(z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(),
                                                z.data_ptr(), 64, 32, 8, 128, 128, 256, 16, cabi.stream(dev))
    assert code == -4
    assert b"scratch" in lib.aops_strerror(code)
