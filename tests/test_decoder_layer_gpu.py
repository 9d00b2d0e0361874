"""One decoder layer chained from the operators in the order of the reference's graph builder
(csrc/ffi/graph.cpp:145-181 add_decoder_layer, :205-290 add_attn, add_mlp), against a plain fp32 torch
layer built on the oracle.  Linear layers run as grouped_matmul with one expert (the reference uses the
vendor's Linear there); the per-head q/k RMSNorm runs as add_rms_norm with a zero residual."""
import pytest
import torch

import oracle.ops_ref as R

pytestmark = pytest.mark.gpu
H = torch.float16


def _linear_dev(ops, x, w_nk, gl):
    # w_nk: [N, K] storage; the operator takes the logical [1, K, N] view of it
    return ops.grouped_matmul(x, w_nk[None].transpose(1, 2), gl)


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("Hq,Hkv,D", [(8, 2, 128), (6, 2, 64)])
def test_decoder_layer_decode_step(ops, dev, fused, Hq, Hkv, D):
    import ascend910a_extras.fused as F

    torch.manual_seed(1)
    B, P, NB, inter, eps = 6, 32, 40, 1024, 1e-6
    hidden = 512
    q_size, kv_size = Hq * D, Hkv * D
    ctx = torch.tensor([1, 31, 32, 33, 100, 257], dtype=torch.int32)       # context lengths including the new token
    max_pages = 10
    perm = torch.randperm(NB)
    bt = torch.zeros(B, max_pages, dtype=torch.int32)
    c = 0
    for b in range(B):
        npg = (int(ctx[b]) + P - 1) // P
        bt[b, :npg] = perm[c:c + npg].int()
        c += npg
    pos = (ctx - 1).int()
    slots = torch.tensor([int(bt[b, int(pos[b]) // P]) * P + int(pos[b]) % P for b in range(B)], dtype=torch.int32)
    kc = torch.randn(NB, kv_size // 16, P, 16).half()
    vc = torch.randn(NB, kv_size // 16, P, 16).half()
    cos, sin = R.build_cos_sin_cache(512, D, theta=1e6)

    x = torch.randn(B, hidden).half()
    res_in = torch.randn(B, hidden).half()
    w_ln1 = (1 + 0.1 * torch.randn(hidden)).half()
    w_ln2 = (1 + 0.1 * torch.randn(hidden)).half()
    w_qn = (1 + 0.1 * torch.randn(D)).half()
    w_kn = (1 + 0.1 * torch.randn(D)).half()
    w_qkv = (torch.randn(q_size + 2 * kv_size, hidden) / hidden ** 0.5).half()
    w_o = (torch.randn(hidden, q_size) / q_size ** 0.5).half()
    w_gu = (torch.randn(2 * inter, hidden) / hidden ** 0.5).half()
    w_dn = (torch.randn(hidden, inter) / inter ** 0.5).half()

    # ---------------- device chain
    d = lambda t: t.to(dev)
    gl = torch.tensor([B], dtype=torch.int64, device=dev)
    kcd, vcd = d(kc), d(vc)
    hs, res = ops.add_rms_norm(d(x), d(res_in), d(w_ln1), eps)
    qkv = _linear_dev(ops, hs, d(w_qkv), gl)
    q, k, v = qkv.split([q_size, kv_size, kv_size], dim=-1)
    v3 = v.reshape(B, Hkv, D).contiguous()
    if fused:   # q/k norm + rope + cache write in one launch
        oq = F.rope_reshape_and_cache(q.reshape(B, Hq, D).contiguous(), k.reshape(B, Hkv, D).contiguous(), v3, d(pos),
                                      d(cos), d(sin), kcd, vcd, d(slots), q_norm_weight=d(w_qn), k_norm_weight=d(w_kn),
                                      epsilon=eps)
    else:
        zq = torch.zeros(B * Hq, D, dtype=H, device=dev)
        zk = torch.zeros(B * Hkv, D, dtype=H, device=dev)
        qn = ops.add_rms_norm(q.reshape(B * Hq, D).contiguous(), zq, d(w_qn), eps)[0].view(B, Hq, D)
        kn = ops.add_rms_norm(k.reshape(B * Hkv, D).contiguous(), zk, d(w_kn), eps)[0].view(B, Hkv, D)
        oq, ok = ops.rope(qn, kn, d(pos), d(cos), d(sin))
        ops.reshape_and_cache(ok, v3, kcd, vcd, d(slots))
    attn = ops.paged_attention(oq, kcd, vcd, d(bt), d(ctx))
    o = _linear_dev(ops, attn.reshape(B, q_size), d(w_o), gl)
    hs2, res2 = ops.add_rms_norm(o, res, d(w_ln2), eps)
    if fused:
        act = F.grouped_matmul_swiglu(hs2, d(w_gu)[None].transpose(1, 2), gl)
    else:
        act = ops.swiglu(_linear_dev(ops, hs2, d(w_gu), gl))
    y = _linear_dev(ops, act, d(w_dn), gl)

    # ---------------- fp32 reference on the CPU (oracle functions for the operators, fp32 matmuls)
    def rms(t, w):
        t = t.float()
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w.float()

    t1 = x.float() + res_in.float()
    r_hs = rms(t1, w_ln1)
    r_qkv = r_hs @ w_qkv.float().T
    rq, rk, rv = r_qkv.split([q_size, kv_size, kv_size], dim=-1)
    rq = rms(rq.reshape(B, Hq, D), w_qn)
    rk = rms(rk.reshape(B, Hkv, D), w_kn)
    rq_r, rk_r = R.rope_ref(rq.half(), rk.half(), pos, cos, sin)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    R.reshape_and_cache_ref(rk_r, kc_ref, slots, rv.reshape(B, Hkv, D).half(), vc_ref)
    r_attn = R.paged_attention_ref(rq_r, kc_ref, vc_ref, bt, ctx).float()
    r_o = r_attn.reshape(B, q_size) @ w_o.float().T
    t2 = r_o + t1
    r_hs2 = rms(t2, w_ln2)
    r_h = r_hs2 @ w_gu.float().T
    r_act = torch.nn.functional.silu(r_h[:, :inter]) * r_h[:, inter:]
    r_y = r_act @ w_dn.float().T

    # the residual stream and the layer output, both O(1): a few fp16 roundings deep
    torch.testing.assert_close(res2.cpu().float(), t2, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(y.cpu().float(), r_y, rtol=3e-2, atol=3e-2)
    # the cache now holds the new token of every sequence: its v row is the projected v, bit for bit
    for b in range(B):
        rows = R.gather_kv_from_cache(vcd.cpu(), bt[b], int(ctx[b]), Hkv)
        assert torch.equal(rows[-1], v3[b].cpu())
