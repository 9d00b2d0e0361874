#!/usr/bin/env python3
"""Benchmark of the ascend910a_extras operator set on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--ops all|norm|cache|rope|mlp|moe|moe_gate_up|moe_down|pa_more|dense|gmm_probe|gmm_probe_gate_up|gmm_probe_down|gmm_probe_dense|scaled,...] [--no-cpu]

A "step" is one paged_attention decode call over the batch of BASELINE.json configs[4]
(64 sequences, 32 query / 8 kv heads, head_dim 128, contexts ~U[512, 4096], block 128): the
largest HBM-bound workload of the operator set and the one the printed `value` is quoted on.
Every other configuration is measured as well (add_rms_norm, reshape_and_cache, swiglu and the two
dense GEMMs of the MLP, the MoE grouped GEMMs, rope, further paged-attention batches, a compute-bound
dense product, plus clearly labelled scaled shapes of the small operators): the full records go out as
one `{"per_op": [...]}` JSON line BEFORE the headline, and a compact list of them
(`roofline.per_kernel`: operator, config, microseconds, fraction of the bounding peak, CPU ms) sits inside
the headline, which is the last line printed.

Timing:
  * `ms_per_step` / `value`: wall clock around exactly K eager steps through the Python API,
    bracketed by torch.cuda.synchronize() on both sides, inputs resident in HBM.
  * `roofline` and `per_op[*].gpu_us`: HIP events (on the stream the kernels are launched on)
    around replays of a HIP graph that holds one launch per rotating buffer set, so that
    back-to-back kernels are timed rather than the host's launch rate; the buffer sets are
    sized so that the footprint between two uses of the same buffer exceeds the 256 MB Infinity
    Cache.  Algorithmic bytes = every input read once, every output written once.
  * `cpu_baseline` / `per_op[*].cpu_ms`: the CPU oracle (plain torch, fp32 math) on the same
    inputs on this machine's host cores: one warm-up run, then the median of three timed runs.
    The oracle is the checker and the timed baseline only; nothing measured on the GPU goes
    through it.
  * `launch_floor_us`: an empty kernel with the operator's launch geometry through the same
    graph-replay timer: what a latency-bound operator is up against besides HBM.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "ascend-ops_amd"), os.path.join(ROOT, "include")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published
CACHE_BYTES = 320 << 20      # Infinity Cache (256 MB) + L2, what a rotation has to exceed


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# --------------------------------------------------------------------------------------- timing
def _events_ms(fn, reps):
    import torch

    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1)


def time_graph(calls, min_launches=200, trials=5):
    """Per-launch GPU time (microseconds) of `calls` (one closure per buffer set), measured with
    HIP events around replays of a graph that holds every closure once."""
    import torch

    for c in calls:
        c()
    torch.cuda.synchronize()
    # at least 32 launches per graph: the gap between two replays is then shared by many launches
    rounds = max(1, -(-32 // len(calls)))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(rounds):
            for c in calls:
                c()
    launches = rounds * len(calls)
    reps = max(1, -(-min_launches // launches))
    graph.replay()
    per = []
    for _ in range(trials):
        per.append(_events_ms(graph.replay, reps) * 1e3 / (reps * launches))
    del graph
    return statistics.median(per), min(per)


def time_eager(calls, warmup, iters):
    import torch

    n = len(calls)
    for i in range(warmup):
        calls[i % n]()
    it = iter(range(10**9))
    ms = _events_ms(lambda: calls[next(it) % n](), iters)
    return ms * 1e3 / iters


CPU_RUNS = 3


def time_cpu(fn, runs=CPU_RUNS):
    """One warm-up run, then the median of `runs` timed ones (milliseconds); returns (ms, last result)."""
    out = fn()
    ts = []
    for _ in range(runs):
        t0 = time.perf_counter()
        out = fn()
        ts.append(time.perf_counter() - t0)
    return statistics.median(ts) * 1e3, out


def n_sets_for(bytes_per_set, lo=2, hi=128):
    return int(max(lo, min(hi, math.ceil(CACHE_BYTES / max(bytes_per_set, 1)) + 1)))


# --------------------------------------------------------------------------------------- C ABI
class Lib:
    """Direct C-ABI launches on preallocated buffers (kernel timing without allocator effects)."""

    def __init__(self):
        import torch
        import cabi  # include/cabi.py: libaops.so through ctypes, signatures parsed from include/aops.h

        self.lib = cabi.lib()
        self.torch = torch

    def stream(self):
        return self.torch.cuda.current_stream().cuda_stream

    def check(self, code):
        if code != 0:
            raise RuntimeError(self.lib.aops_strerror(code).decode())

    def launch_floor_us(self, workgroups, threads):
        """Per-launch time of an empty kernel with this geometry, through the timer the operators use."""
        med, _ = time_graph([lambda: self.check(self.lib.aops_empty_launch(workgroups, threads, self.stream()))])
        return round(med, 3)


def entry(op, config, shape, bound, alg_bytes, alg_flops, gpu_us, gpu_us_min, eager_us, cpu_ms, cores, note=None):
    e = {
        "op": op, "config": config, "shape": shape, "bound": bound,
        "algorithmic_bytes": alg_bytes, "algorithmic_flops": alg_flops,
        "gpu_us": round(gpu_us, 3), "gpu_us_min": round(gpu_us_min, 3),
        "api_eager_us": None if eager_us is None else round(eager_us, 3),
    }
    gbps = alg_bytes / (gpu_us * 1e-6) / 1e9
    e["GBps"] = round(gbps, 1)
    e["hbm_frac"] = round(gbps / HBM_PEAK_GBPS, 4)
    if alg_flops:
        tf = alg_flops / (gpu_us * 1e-6) / 1e12
        e["TFLOPs"] = round(tf, 1)
        e["mfma_frac"] = round(tf / MFMA_F16_PEAK_TFLOPS, 4)
    if cpu_ms is not None:
        e["cpu_ms"] = round(cpu_ms, 3)
        e["cpu_cores"] = cores
        e["cpu_runs"] = f"1 warm-up + median of {CPU_RUNS}"
        e["gpu_over_cpu"] = round(cpu_ms * 1e3 / gpu_us, 1)
    if note:
        e["note"] = note
    return e


# --------------------------------------------------------------------------------------- workloads
def bench_add_rms_norm(L, ops, R, dev, cpu, T, config, note=None, floor=False):
    import torch

    Hd, eps = 4096, 1e-6
    torch.manual_seed(0)
    x = torch.randn(T, Hd).half()
    r = torch.randn(T, Hd).half()
    w = (1 + 0.1 * torch.randn(Hd)).half()
    alg = 4 * T * Hd * 2 + Hd * 2
    n = n_sets_for(alg)
    xs = [x.to(dev).clone() for _ in range(n)]
    rs = [r.to(dev).clone() for _ in range(n)]
    ys = [torch.empty_like(xs[0]) for _ in range(n)]
    os_ = [torch.empty_like(xs[0]) for _ in range(n)]
    wd = w.to(dev)

    def mk(i):
        return lambda: L.check(L.lib.aops_add_rms_norm_f16(xs[i].data_ptr(), rs[i].data_ptr(), wd.data_ptr(), eps,
                                                          ys[i].data_ptr(), os_[i].data_ptr(), T, Hd, L.stream()))

    calls = [mk(i) for i in range(n)]
    med, mn = time_graph(calls)
    eager = time_eager([(lambda i=i: ops.add_rms_norm(xs[i], rs[i], wd, eps)) for i in range(n)], 10, 100)
    y_ref, res_ref = R.add_rms_norm_ref(x, r, w, eps)
    torch.testing.assert_close(ys[-1].cpu().float(), y_ref.float(), rtol=1e-2, atol=1e-2)
    assert torch.equal(os_[-1].cpu(), res_ref)
    cpu_ms = time_cpu(lambda: R.add_rms_norm_ref(x, r, w, eps))[0] if cpu else None
    e = entry("add_rms_norm", config, f"x,residual [{T},{Hd}] f16", "hbm", alg, 0, med, mn, eager, cpu_ms,
              torch.get_num_threads(), note)
    if floor:
        e["launch_floor_us"] = L.launch_floor_us(T, 512)  # one workgroup of 512 threads per row
    return e


def bench_swiglu(L, ops, R, dev, cpu, T, d, config, note=None, floor=False):
    import torch

    torch.manual_seed(0)
    x = torch.randn(T, 2 * d).half()
    alg = T * d * 2 * 3
    n = n_sets_for(alg)
    xs = [x.to(dev).clone() for _ in range(n)]
    ys = [torch.empty(T, d, dtype=torch.float16, device=dev) for _ in range(n)]

    def mk(i):
        return lambda: L.check(L.lib.aops_swiglu_f16(xs[i].data_ptr(), ys[i].data_ptr(), T, d, L.stream()))

    med, mn = time_graph([mk(i) for i in range(n)])
    eager = time_eager([(lambda i=i: ops.swiglu(xs[i])) for i in range(n)], 10, 100)
    torch.testing.assert_close(ys[-1].cpu().float(), R.swiglu_ref(x).float(), rtol=1e-2, atol=1e-2)
    cpu_ms = time_cpu(lambda: R.swiglu_ref(x))[0] if cpu else None
    e = entry("swiglu", config, f"x [{T},{2 * d}] f16", "hbm", alg, 0, med, mn, eager, cpu_ms,
              torch.get_num_threads(), note)
    if floor:
        e["launch_floor_us"] = L.launch_floor_us((T * d // 8 + 511) // 512, 256)  # 2 x 16 bytes of output per thread
    return e


def bench_rope(L, ops, R, dev, cpu, B, config, note=None, floor=False):
    import torch

    Hq, Hkv, D, max_pos = 32, 8, 128, 4096
    torch.manual_seed(0)
    q = torch.randn(B, Hq, D).half()
    k = torch.randn(B, Hkv, D).half()
    pos = torch.randint(511, 4096, (B,), dtype=torch.int32)
    cos, sin = R.build_cos_sin_cache(max_pos, D, theta=1e6)
    alg = 2 * B * (Hq + Hkv) * D * 2 + B * 4 + 2 * B * (D // 2) * 2
    n = n_sets_for(alg)
    qs = [q.to(dev).clone() for _ in range(n)]
    ks = [k.to(dev).clone() for _ in range(n)]
    oq = [torch.empty_like(qs[0]) for _ in range(n)]
    ok = [torch.empty_like(ks[0]) for _ in range(n)]
    pd, cd, sd = pos.to(dev), cos.to(dev), sin.to(dev)

    def mk(i):
        return lambda: L.check(L.lib.aops_rope_neox_f16(qs[i].data_ptr(), ks[i].data_ptr(), pd.data_ptr(), cd.data_ptr(),
                                                       sd.data_ptr(), oq[i].data_ptr(), ok[i].data_ptr(), B, Hq, Hkv, D,
                                                       L.stream()))

    med, mn = time_graph([mk(i) for i in range(n)])
    eager = time_eager([(lambda i=i: ops.rope(qs[i], ks[i], pd, cd, sd)) for i in range(n)], 10, 100)
    rq, rk = R.rope_ref(q, k, pos, cos, sin)
    torch.testing.assert_close(oq[-1].cpu().float(), rq.float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(ok[-1].cpu().float(), rk.float(), rtol=1e-2, atol=1e-2)
    cpu_ms = time_cpu(lambda: R.rope_ref(q, k, pos, cos, sin))[0] if cpu else None
    e = entry("rope", config, f"q [{B},{Hq},{D}], k [{B},{Hkv},{D}] f16", "hbm", alg, 0, med, mn, eager, cpu_ms,
              torch.get_num_threads(), note)
    if floor:
        e["launch_floor_us"] = L.launch_floor_us((B * (Hq + Hkv) * D // 16 + 255) // 256, 256)  # 8 pairs per thread
    return e


def bench_reshape_and_cache(L, ops, R, dev, cpu, T, config, note=None, consecutive=False, floor=False):
    import torch

    Hkv, D, NB, P = 8, 128, 1024, 128
    torch.manual_seed(0)
    key = torch.randn(T, Hkv, D).half()
    value = torch.randn(T, Hkv, D).half()
    if consecutive:  # a prefill: every sequence of 512 tokens fills four pages in order, the pages are scattered
        pages = torch.randperm(NB)[: T // P]
        slots = (pages[:, None] * P + torch.arange(P)[None, :]).reshape(-1).int()
    else:
        slots = torch.randperm(NB * P)[:T].int()
    alg = 4 * T * Hkv * D * 2 + T * 4
    n = n_sets_for(alg, lo=2, hi=48)
    n_cache = 2  # 2 x (2 x 256 MiB): a cache pair is reused only after 1 GiB of other lines
    ks = [key.to(dev).clone() for _ in range(n)]
    vs = [value.to(dev).clone() for _ in range(n)]
    kcs = [torch.zeros(NB, Hkv * D // 16, P, 16, dtype=torch.float16, device=dev) for _ in range(n_cache)]
    vcs = [torch.zeros(NB, Hkv * D // 16, P, 16, dtype=torch.float16, device=dev) for _ in range(n_cache)]
    sd = slots.to(dev)

    def mk(i):
        c = i % n_cache
        return lambda: L.check(L.lib.aops_reshape_and_cache_f16(ks[i].data_ptr(), vs[i].data_ptr(), kcs[c].data_ptr(),
                                                               vcs[c].data_ptr(), sd.data_ptr(), T, Hkv * D, NB, P,
                                                               L.stream()))

    med, mn = time_graph([mk(i) for i in range(n)])
    eager = time_eager([(lambda i=i: ops.reshape_and_cache(ks[i], vs[i], kcs[i % n_cache], vcs[i % n_cache], sd))
                        for i in range(n)], 10, 100)
    kc_ref = torch.zeros(NB, Hkv * D // 16, P, 16, dtype=torch.float16)
    vc_ref = torch.zeros_like(kc_ref)
    cpu_ms = None
    if cpu:
        cpu_ms = time_cpu(lambda: R.reshape_and_cache_ref(key, kc_ref, slots, value, vc_ref))[0]
    else:
        R.reshape_and_cache_ref(key, kc_ref, slots, value, vc_ref)
    assert torch.equal(kcs[0].cpu(), kc_ref) and torch.equal(vcs[0].cpu(), vc_ref), "reshape_and_cache not bit-exact"
    e = entry("reshape_and_cache", config, f"key,value [{T},{Hkv},{D}] -> caches [{NB},{Hkv * D // 16},{P},16] f16",
              "hbm", alg, 0, med, mn, eager, cpu_ms, torch.get_num_threads(), note)
    if floor:
        e["launch_floor_us"] = L.launch_floor_us(2 * ((T * Hkv * D // 8 + 255) // 256), 256)  # 16 bytes per thread, K and V
    return e


def _gmm_entry(L, ops, R, dev, cpu, op, config, x, w_storage, gl, note=None, check_rows=4096):
    """x [rows,K] cpu f16, w_storage [E,N,K] cpu f16, gl int64 cumulative."""
    import torch

    rows, K = x.shape
    E, N, _ = w_storage.shape
    end = int(gl[-1])
    flops = 2 * end * K * N
    alg = rows * K * 2 + E * N * K * 2 + end * N * 2 + E * 8
    xd, wd, gd = x.to(dev), w_storage.to(dev), gl.to(dev)
    n = n_sets_for(alg, lo=1, hi=8)
    xs = [xd] + [xd.clone() for _ in range(n - 1)]
    ws = [wd] + [wd.clone() for _ in range(n - 1)]
    ys = [torch.empty(rows, N, dtype=torch.float16, device=dev) for _ in range(n)]

    # what ops.grouped_matmul does: the two-phase entry (one expert with few rows and a long k wants scratch)
    ws_bytes = L.lib.aops_grouped_matmul_workspace(rows, K, E, N)
    scratch = [torch.empty(ws_bytes, dtype=torch.uint8, device=dev) for _ in range(n)] if ws_bytes else None

    def mk(i):
        return lambda: L.check(L.lib.aops_grouped_matmul_ws_f16(
            xs[i].data_ptr(), ws[i].data_ptr(), gd.data_ptr(), ys[i].data_ptr(),
            scratch[i].data_ptr() if ws_bytes else None, ws_bytes, rows, K, E, N, L.stream()))

    med, mn = time_graph([mk(i) for i in range(n)], min_launches=40)
    if ws_bytes:
        note = (note + "; " if note else "") + (
            f"two kernels per call: k range split over the workgroups of a tile ({ws_bytes / 1e6:.1f} MB of fp32 "
            "partial results) + reduction")
    eager = time_eager([(lambda i=i: ops.grouped_matmul(xs[i], ws[i].transpose(1, 2), gd)) for i in range(n)], 3, 20)
    w_logical = w_storage.transpose(1, 2)
    cpu_ms = None
    if cpu:
        cpu_ms, ref = time_cpu(lambda: R.grouped_matmul_ref(x, w_logical, gl))
        torch.testing.assert_close(ys[-1].cpu()[:end].float(), ref[:end].float(), rtol=2e-2, atol=2e-2)
    else:
        # check a slice of rows only (first experts) to keep the run short
        sub_end = min(end, check_rows)
        e_hi = int((gl < sub_end).sum()) + 1
        gsub = torch.clamp(gl[:e_hi], max=sub_end)
        ref = R.grouped_matmul_ref(x[:sub_end], w_logical[:e_hi], gsub)
        torch.testing.assert_close(ys[-1].cpu()[:sub_end].float(), ref.float(), rtol=2e-2, atol=2e-2)
    e = entry(op, config, f"x [{rows},{K}] @ w [{E},{K},{N}] f16", "mfma", alg, flops, med, mn, eager, cpu_ms,
              torch.get_num_threads(), note)
    hbm_floor_us = alg / (HBM_PEAK_GBPS * 1e9) * 1e6
    mfma_floor_us = flops / (MFMA_F16_PEAK_TFLOPS * 1e12) * 1e6
    e["hbm_floor_us"] = round(hbm_floor_us, 2)
    e["mfma_floor_us"] = round(mfma_floor_us, 2)
    e["frac_of_roofline_ceiling"] = round(max(hbm_floor_us, mfma_floor_us) / med, 4)
    return e, ys[-1]


def _gmm_swiglu_entry(L, ops, dev, config, x, w_storage, gl, h_dev):
    """Fused gate_up + SwiGLU (extension, no reference counterpart): timed like the other GEMMs and
    checked against the device's own two-operator chain (which is checked against the oracle)."""
    import torch

    rows, K = x.shape
    E, N, _ = w_storage.shape
    end = int(gl[-1])
    flops = 2 * end * K * N
    alg = rows * K * 2 + E * N * K * 2 + end * (N // 2) * 2 + E * 8
    xd, wd, gd = x.to(dev), w_storage.to(dev), gl.to(dev)
    n = n_sets_for(alg, lo=1, hi=8)
    xs = [xd] + [xd.clone() for _ in range(n - 1)]
    ws = [wd] + [wd.clone() for _ in range(n - 1)]
    ys = [torch.empty(rows, N // 2, dtype=torch.float16, device=dev) for _ in range(n)]

    def mk(i):
        return lambda: L.check(L.lib.aops_grouped_matmul_swiglu_f16(xs[i].data_ptr(), ws[i].data_ptr(), gd.data_ptr(),
                                                                   ys[i].data_ptr(), rows, K, E, N, L.stream()))

    med, mn = time_graph([mk(i) for i in range(n)], min_launches=40)
    two = ops.swiglu(h_dev)
    torch.testing.assert_close(ys[-1][:end].float(), two[:end].float(), rtol=2e-2, atol=2e-2)
    e = entry("grouped_matmul_swiglu", config, f"x [{rows},{K}] @ w [{E},{K},{N}] f16 -> [{rows},{N // 2}]", "mfma", alg,
              flops, med, mn, None, None, torch.get_num_threads(),
              "extension: activation fused into the GEMM epilogue, replaces the gate_up and swiglu lines above")
    return e


def _gmm_swiglu_gather_entry(L, dev, w_storage, tokens, topk):
    """Fused gate_up + SwiGLU that also reads its rows through the routing order (extension): x stays in token
    order [tokens, hidden]; checked bit for bit against the explicit gather followed by the fused kernel."""
    import torch
    import ascend910a_extras.ascend910a_extras_C as C
    import ascend910a_extras.moe as moe

    E, N, K = w_storage.shape
    rows = tokens * topk
    torch.manual_seed(2)
    ids = torch.randint(0, E, (tokens, topk), dtype=torch.int32).to(dev)
    x = torch.randn(tokens, K).half().to(dev)
    wd = w_storage.to(dev)
    s_idx, _, gl = moe.moe_sort(ids, E)
    flops = 2 * rows * K * N
    alg = tokens * K * 2 + E * N * K * 2 + rows * (N // 2) * 2 + rows * 4 + E * 8
    y = torch.empty(rows, N // 2, dtype=torch.float16, device=dev)
    call = lambda: L.check(L.lib.aops_grouped_matmul_swiglu_gather_f16(x.data_ptr(), s_idx.data_ptr(), topk, tokens,
                                                                       wd.data_ptr(), gl.data_ptr(), y.data_ptr(), rows, K, E, N,
                                                                       L.stream()))
    med, mn = time_graph([call], min_launches=40)
    want = C.grouped_matmul_swiglu(moe.moe_gather(x, s_idx, gl, topk), wd.transpose(1, 2), gl)
    assert torch.equal(y, want)
    return entry("grouped_matmul_swiglu_gather", "4: MoE gate_up + activation + row gather, fused",
                 f"x [{tokens},{K}] (token order, top-{topk}) @ w [{E},{K},{N}] f16 -> [{rows},{N // 2}]", "mfma", alg, flops,
                 med, mn, None, None, 1,
                 "extension: replaces moe_gather + gate_up + swiglu; one weight set, so the weights are re-read from HBM every launch but x (17 MB) stays cached")


def _moe_mlp_entry(dev, w1_storage, w2_storage, tokens, topk, decode=False):
    """The whole routed expert MLP of configs[3] through the extension API (sort -> gate_up with gather and SwiGLU
    -> down -> combine), captured in one HIP graph: what the operators add up to for a caller."""
    import torch
    import ascend910a_extras.moe as moe

    E, N1, K = w1_storage.shape
    torch.manual_seed(3)
    x = torch.randn(tokens, K).half().to(dev)
    logits = torch.randn(tokens, E)
    wts, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
    wts = (wts / wts.sum(-1, keepdim=True)).float().to(dev)
    ids = ids.int().to(dev)
    w1 = w1_storage.to(dev).transpose(1, 2)
    w2 = w2_storage.to(dev).transpose(1, 2)
    for _ in range(2):
        out = moe.moe_mlp(x, ids, wts, w1, w2)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = moe.moe_mlp(x, ids, wts, w1, w2)
    graph.replay()
    torch.cuda.synchronize()
    trials = []
    for _ in range(5):
        trials.append(_events_ms(graph.replay, 10) * 1e3 / 10)
    trials.sort()
    flops = 2 * tokens * topk * K * N1 + 2 * tokens * topk * (N1 // 2) * K
    if decode:
        # a decode step: the weights of every expert that is hit are streamed once, the arithmetic is negligible
        hit = int(torch.unique(ids).numel())
        wbytes = hit * (N1 * K + K * (N1 // 2)) * 2
        e = {"op": "moe_mlp", "config": f"4 at decode size ({tokens} tokens): routed expert MLP end to end (extension)",
             "shape": f"x [{tokens},{K}], top-{topk} of {E} experts ({hit} hit), inter {N1 // 2}", "bound": "hbm",
             "algorithmic_bytes": wbytes, "gpu_us": round(trials[len(trials) // 2], 3), "gpu_us_min": round(trials[0], 3)}
        e["GBps"] = round(wbytes / e["gpu_us"] / 1e3, 1)
        e["hbm_frac"] = round(e["GBps"] / HBM_PEAK_GBPS, 4)
        e["note"] = "weight-stream bound: bytes = the fp16 weights of the experts that are hit"
        return e
    e = {"op": "moe_mlp", "config": "4: routed expert MLP end to end (extension, five launches in one graph)",
         "shape": f"x [{tokens},{K}], top-{topk} of {E} experts, inter {N1 // 2}", "bound": "mfma",
         "algorithmic_flops": flops, "gpu_us": round(trials[len(trials) // 2], 3), "gpu_us_min": round(trials[0], 3)}
    e["TFLOPs"] = round(flops / e["gpu_us"] / 1e6, 1)
    e["mfma_frac"] = round(e["TFLOPs"] / MFMA_F16_PEAK_TFLOPS, 4)
    return e


def _moe_glue_entries(L, dev, E, hidden, tokens, topk):
    """Routing glue of the expert MLP at the configs[3] shape (extension, no reference operator): device-side
    stable sort -> group_list, row gather, weighted combine.  Checked against the oracle in tests/test_moe_gpu.py."""
    import torch
    import ascend910a_extras.moe as moe

    torch.manual_seed(1)
    n = tokens * topk
    ids = torch.randint(0, E, (tokens, topk), dtype=torch.int32).to(dev)
    wts = torch.rand(tokens, topk).to(dev)
    x = torch.randn(tokens, hidden).half().to(dev)
    ws_bytes = L.lib.aops_moe_sort_workspace(n, E)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    s_idx = torch.empty(n, dtype=torch.int32, device=dev)
    inv = torch.empty(n, dtype=torch.int32, device=dev)
    gl = torch.empty(E, dtype=torch.int64, device=dev)
    out = []
    sort_call = lambda: L.check(L.lib.aops_moe_sort_i32(ids.data_ptr(), n, E, s_idx.data_ptr(), inv.data_ptr(),
                                                        gl.data_ptr(), ws.data_ptr(), ws_bytes, L.stream()))
    med, mn = time_graph([sort_call], min_launches=100)
    out.append(entry("moe_sort", "4: routing sort (extension)", f"ids [{tokens},{topk}] int32, {E} experts", "hbm",
                     n * 4 * 3 + E * 8, 0, med, mn, None, None, 1, "two launches: per-slice histograms, then a scatter whose waves scan the histograms themselves (stable)"))
    n_sets = n_sets_for(n * hidden * 2 * 2)
    xs = [torch.empty(n, hidden, dtype=torch.float16, device=dev) for _ in range(n_sets)]
    med, mn = time_graph([(lambda i=i: L.check(L.lib.aops_moe_gather_f16(x.data_ptr(), s_idx.data_ptr(), gl.data_ptr(),
                                                                         xs[i].data_ptr(), n, topk, hidden, E, L.stream())))
                          for i in range(n_sets)])
    out.append(entry("moe_gather", "4: row gather into expert order (extension)", f"x [{tokens},{hidden}] -> [{n},{hidden}] f16",
                     "hbm", tokens * hidden * 2 + n * hidden * 2 + n * 4, 0, med, mn, None, None, 1))
    outs = [torch.empty(tokens, hidden, dtype=torch.float16, device=dev) for _ in range(n_sets)]
    med, mn = time_graph([(lambda i=i: L.check(L.lib.aops_moe_combine_f16(xs[i].data_ptr(), inv.data_ptr(), wts.data_ptr(),
                                                                          ids.data_ptr(), outs[i].data_ptr(), tokens, topk,
                                                                          hidden, E, L.stream())))
                          for i in range(n_sets)])
    out.append(entry("moe_combine", "4: weighted combine to token order (extension)",
                     f"y [{n},{hidden}] -> [{tokens},{hidden}] f16", "hbm",
                     n * hidden * 2 + tokens * hidden * 2 + n * 12, 0, med, mn, None, None, 1))
    return out


def bench_moe(L, ops, R, dev, cpu):
    import torch

    E, hidden, inter, tokens, topk = 128, 2048, 768, 4096, 8
    torch.manual_seed(0)
    rows = tokens * topk
    ids = torch.randint(0, E, (rows,))
    gl = R.make_group_list(ids, E)
    x = torch.randn(rows, hidden).half()
    w1 = torch.empty(E, 2 * inter, hidden, dtype=torch.float16)
    w2 = torch.empty(E, hidden, inter, dtype=torch.float16)
    for e in range(E):  # chunked generation keeps the fp32 temporaries small
        w1[e] = (0.02 * torch.randn(2 * inter, hidden)).half()
        w2[e] = (0.02 * torch.randn(hidden, inter)).half()
    out = []
    e1, h_dev = _gmm_entry(L, ops, R, dev, cpu, "grouped_matmul", "4: MoE gate_up", x, w1, gl)
    out.append(e1)
    e_fused = _gmm_swiglu_entry(L, ops, dev, "4: MoE gate_up + activation, fused", x, w1, gl, h_dev)
    e_gather = _gmm_swiglu_gather_entry(L, dev, w1, tokens, topk)
    e_layer = _moe_mlp_entry(dev, w1, w2, tokens, topk)
    e_decode = _moe_mlp_entry(dev, w1, w2, 64, topk, decode=True)
    del w1
    h = ops.swiglu(h_dev)
    # swiglu at the MoE shape
    T, d = rows, inter
    alg = T * d * 2 * 3
    n = n_sets_for(alg)
    hs = [h_dev.clone() for _ in range(n)]
    ys = [torch.empty(T, d, dtype=torch.float16, device=dev) for _ in range(n)]
    med, mn = time_graph([(lambda i=i: L.check(L.lib.aops_swiglu_f16(hs[i].data_ptr(), ys[i].data_ptr(), T, d, L.stream())))
                          for i in range(n)])
    h_cpu = h_dev.cpu()
    cpu_ms = time_cpu(lambda: R.swiglu_ref(h_cpu))[0] if cpu else None
    torch.testing.assert_close(ys[-1].cpu().float(), R.swiglu_ref(h_cpu).float(), rtol=1e-2, atol=1e-2)
    out.append(entry("swiglu", "4: MoE activation", f"x [{T},{2 * d}] f16", "hbm", alg, 0, med, mn, None, cpu_ms,
                     torch.get_num_threads()))
    del hs, ys
    e2, _ = _gmm_entry(L, ops, R, dev, cpu, "grouped_matmul", "4: MoE down", h.cpu(), w2, gl)
    out.append(e2)
    out.append(e_fused)
    out.append(e_gather)
    out.append(e_layer)
    out.append(e_decode)
    out.extend(_moe_glue_entries(L, dev, E, hidden, tokens, topk))
    tot_flops = e1["algorithmic_flops"] + e2["algorithmic_flops"]
    tot_us = e1["gpu_us"] + e2["gpu_us"]
    out.append({
        "op": "grouped_matmul", "config": "4: MoE gate_up + down (sum of the two GEMMs)",
        "algorithmic_flops": tot_flops, "gpu_us": round(tot_us, 3),
        "TFLOPs": round(tot_flops / tot_us / 1e6, 1),
        "mfma_frac": round(tot_flops / tot_us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4),
    })
    return out


def bench_moe_one(L, ops, R, dev, which):
    """One GEMM of configs[3] by itself (for profiler runs that must tell the two apart): gate_up on x ~ N(0,1),
    or down on activations of the magnitude the real chain produces."""
    import torch

    E, hidden, inter, tokens, topk = 128, 2048, 768, 4096, 8
    torch.manual_seed(0)
    rows = tokens * topk
    gl = R.make_group_list(torch.randint(0, E, (rows,)), E)
    K, N = (hidden, 2 * inter) if which.startswith("gate_up") else (inter, hidden)
    x = (torch.randn(rows, K) * (1.0 if which.startswith("gate_up") else 0.3)).half()
    w = torch.empty(E, N, K, dtype=torch.float16)
    for e in range(E):
        w[e] = (0.02 * torch.randn(N, K)).half()
    if which.endswith("_padded"):
        return _gmm_padded_entry(L, dev, which, x, w, gl)
    e, _ = _gmm_entry(L, ops, R, dev, False, "grouped_matmul", f"4: MoE {which} (alone)", x, w, gl)
    return e


def _gmm_padded_entry(L, dev, which, x, w, gl):
    """One GEMM of configs[3] over weights whose rows are padded by one cache line (aops_grouped_matmul_ldw_f16), alone in
    its run so that a profiler can tell it from the unpadded launches; checked bit for bit against the unpadded kernel."""
    import torch

    rows, K = x.shape
    E, N, _ = w.shape
    ldw = K + 64
    xd, wd, gd = x.to(dev), w.to(dev), gl.to(dev)
    y_ref = torch.empty(rows, N, dtype=torch.float16, device=dev)
    L.check(L.lib.aops_grouped_matmul_variant_f16(6, xd.data_ptr(), wd.data_ptr(), gd.data_ptr(), y_ref.data_ptr(), rows, K,
                                                  E, N, L.stream()))
    sets = 2
    wps = []
    for _ in range(sets):
        wp = torch.zeros(E, N, ldw, dtype=torch.float16, device=dev)
        wp[:, :, :K] = wd
        wps.append(wp)
    del wd
    xs = [xd, xd.clone()]
    ys = [torch.empty(rows, N, dtype=torch.float16, device=dev) for _ in range(sets)]
    calls = [(lambda i=i: L.check(L.lib.aops_grouped_matmul_ldw_f16(xs[i].data_ptr(), wps[i].data_ptr(), ldw, gd.data_ptr(),
                                                                    ys[i].data_ptr(), rows, K, E, N, L.stream())))
             for i in range(sets)]
    med, mn = time_graph(calls, min_launches=40)
    assert torch.equal(ys[0], y_ref), "padded weight rows must give the same bits"
    end = int(gl[-1])
    return entry("grouped_matmul_ldw", f"4: MoE {which} (alone; weight rows {2 * ldw} bytes apart)",
                 f"x [{rows},{K}] @ w [{E},{K},{N}] f16", "mfma", rows * K * 2 + E * N * K * 2 + end * N * 2 + E * 8,
                 2 * end * K * N, med, mn, None, None, 1)


def bench_mlp(L, ops, R, dev, cpu):
    import torch

    bs, hidden, inter = 256, 4096, 14336
    torch.manual_seed(0)
    x = torch.randn(bs, hidden).half()
    gu = torch.empty(2 * inter, hidden, dtype=torch.float16)
    for i in range(0, 2 * inter, 2048):
        gu[i:i + 2048] = (0.02 * torch.randn(2048, hidden)).half()
    dn = (0.02 * torch.randn(hidden, inter)).half()
    gl = torch.tensor([bs], dtype=torch.int64)
    out = []
    e1, h_dev = _gmm_entry(L, ops, R, dev, cpu, "grouped_matmul (E=1)", "3: MLP gate_up GEMM", x, gu[None], gl,
                           note="dense GEMM run as one expert; weight-stream bound, reported not scored")
    out.append(e1)
    out.append(bench_swiglu(L, ops, R, dev, cpu, bs, inter, "3: MLP swiglu", floor=True))
    h = ops.swiglu(h_dev)
    e2, y_dev = _gmm_entry(L, ops, R, dev, cpu, "grouped_matmul (E=1)", "3: MLP down GEMM", h.cpu(), dn[None], gl,
                           note="dense GEMM run as one expert; weight-stream bound, reported not scored")
    out.append(e2)
    if cpu:
        torch.testing.assert_close(y_dev.cpu().float(), R.mlp_ref(x, gu, dn).float(), rtol=2e-2, atol=2e-2)
    # the same hidden size at a decode batch of 16: a square projection as a pure weight stream (extension)
    xq = torch.randn(16, hidden).half()
    wq = (0.02 * torch.randn(hidden, hidden)).half()
    e3, _ = _gmm_entry(L, ops, R, dev, cpu, "grouped_matmul (E=1)", "3 at decode size: 16 rows, 4096 -> 4096",
                       xq, wq[None], torch.tensor([16], dtype=torch.int64),
                       note="weight-streaming kernel for at most 16 rows (one launch, no workspace); weight-stream bound")
    e3["bound"] = "hbm"
    out.append(e3)
    return out


class PagedAttentionWorkload:
    """BASELINE.json configs[4]: decode attention with neox rope and the cache write of the new token."""

    def __init__(self, R, dev, n_sets=2):
        import torch

        self.B, self.Hq, self.Hkv, self.D, self.P, self.NB = 64, 32, 8, 128, 128, 2304
        B, Hq, Hkv, D, P, NB = self.B, self.Hq, self.Hkv, self.D, self.P, self.NB
        torch.manual_seed(0)
        self.ctx = torch.randint(512, 4097, (B,), dtype=torch.int32)
        pages_per = ((self.ctx + P - 1) // P).tolist()
        self.max_pages = 32
        perm = torch.randperm(NB)
        self.bt = torch.zeros(B, self.max_pages, dtype=torch.int32)
        c = 0
        for b, npg in enumerate(pages_per):
            self.bt[b, :npg] = perm[c:c + npg].int()
            c += npg
        self.q = torch.randn(B, Hq, D).half()
        self.k = torch.randn(B, Hkv, D).half()
        self.v = torch.randn(B, Hkv, D).half()
        self.kc = torch.empty(NB, Hkv * D // 16, P, 16, dtype=torch.float16)
        self.vc = torch.empty_like(self.kc)
        for i in range(0, NB, 64):  # chunked: keeps fp32 temporaries small
            self.kc[i:i + 64] = torch.randn(min(64, NB - i), Hkv * D // 16, P, 16).half()
            self.vc[i:i + 64] = torch.randn(min(64, NB - i), Hkv * D // 16, P, 16).half()
        self.cos, self.sin = R.build_cos_sin_cache(4096, D, theta=1e6)
        self.pos = (self.ctx - 1).int()
        self.slots = torch.tensor([int(self.bt[b, int(self.pos[b]) // P]) * P + int(self.pos[b]) % P for b in range(B)],
                                  dtype=torch.int32)
        sum_ctx = int(self.ctx.sum())
        self.sum_ctx = sum_ctx
        self.alg_bytes = sum_ctx * Hkv * D * 2 * 2 + 2 * B * Hq * D * 2 + self.bt.numel() * 4 + B * 4
        self.dev = dev
        self.d = {}
        for name in ("q", "k", "v", "cos", "sin", "pos", "slots", "bt", "ctx"):
            self.d[name] = getattr(self, name).to(dev)
        kcd, vcd = self.kc.to(dev), self.vc.to(dev)
        self.kcs = [kcd] + [kcd.clone() for _ in range(n_sets - 1)]
        self.vcs = [vcd] + [vcd.clone() for _ in range(n_sets - 1)]
        self.n_sets = n_sets

    def step(self, ops, i=0):
        d = self.d
        return ops.paged_attention(d["q"], self.kcs[i % self.n_sets], self.vcs[i % self.n_sets], d["bt"], d["ctx"])

    def pipeline(self, ops, i=0):
        d = self.d
        oq, ok = ops.rope(d["q"], d["k"], d["pos"], d["cos"], d["sin"])
        ops.reshape_and_cache(ok, d["v"], self.kcs[i % self.n_sets], self.vcs[i % self.n_sets], d["slots"])
        return ops.paged_attention(oq, self.kcs[i % self.n_sets], self.vcs[i % self.n_sets], d["bt"], d["ctx"])

    def pipeline_fused(self, ops, i=0):
        import ascend910a_extras.fused as fused

        d = self.d
        kc, vc = self.kcs[i % self.n_sets], self.vcs[i % self.n_sets]
        oq = fused.rope_reshape_and_cache(d["q"], d["k"], d["v"], d["pos"], d["cos"], d["sin"], kc, vc, d["slots"])
        return ops.paged_attention(oq, kc, vc, d["bt"], d["ctx"])


def bench_paged_attention(L, ops, R, dev, cpu, wl):
    import torch

    B, Hq, Hkv, D, P = wl.B, wl.Hq, wl.Hkv, wl.D, wl.P
    ws_bytes = L.lib.aops_paged_attention_workspace(B, Hq, Hkv, D, P, wl.max_pages)
    wss = [torch.empty(ws_bytes, dtype=torch.uint8, device=dev) for _ in range(wl.n_sets)]
    outs = [torch.empty(B, Hq, D, dtype=torch.float16, device=dev) for _ in range(wl.n_sets)]
    d = wl.d

    def mk(i):
        return lambda: L.check(L.lib.aops_paged_attention_f16(
            d["q"].data_ptr(), wl.kcs[i].data_ptr(), wl.vcs[i].data_ptr(), d["bt"].data_ptr(), d["ctx"].data_ptr(),
            outs[i].data_ptr(), wss[i].data_ptr(), ws_bytes, B, Hq, Hkv, D, P, wl.max_pages, wl.NB, L.stream()))

    med, mn = time_graph([mk(i) for i in range(wl.n_sets)], min_launches=40)
    eager = time_eager([(lambda i=i: wl.step(ops, i)) for i in range(wl.n_sets)], 5, 40)
    cpu_ms = None
    ref = None
    if cpu:
        cpu_ms, ref = time_cpu(lambda: R.paged_attention_ref(wl.q, wl.kc, wl.vc, wl.bt, wl.ctx))
        torch.testing.assert_close(outs[0].cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)
    e = entry("paged_attention", "5: decode attention", f"q [{B},{Hq},{D}], caches [{wl.NB},{Hkv * D // 16},{P},16], "
              f"sum(context)={wl.sum_ctx}", "hbm", wl.alg_bytes, 4 * wl.sum_ctx * Hq * D, med, mn, eager, cpu_ms,
              torch.get_num_threads(), note="one kernel per call: whole sequences per workgroup, longest first, no merge")
    e.pop("TFLOPs", None)
    e.pop("mfma_frac", None)
    # whole decode step: rope -> cache write -> attention (graph of the three C-ABI calls via the API)
    pipe = time_eager([(lambda i=i: wl.pipeline(ops, i)) for i in range(wl.n_sets)], 5, 40)
    e["pipeline_rope_cache_attention_api_eager_us"] = round(pipe, 2)
    pipe2 = time_eager([(lambda i=i: wl.pipeline_fused(ops, i)) for i in range(wl.n_sets)], 5, 40)
    e["pipeline_fused_rope_cache_then_attention_api_eager_us"] = round(pipe2, 2)
    torch.testing.assert_close(wl.pipeline_fused(ops, 0).float(), wl.pipeline(ops, 0).float(), rtol=0, atol=0)
    return e



def bench_pa_shape(L, R, dev, cpu, config, lens, Hq, Hkv, D, P, max_pages, note):
    """Paged attention on another batch shape through the C ABI: graph-timed, oracle-checked.  These lines cover
    what the headline batch does not run: the balanced partition (pa_decode_balanced) for up to 64 and for more
    sequences, the merge (pa_decode_merge), other head sizes, wide groups of query heads and the generic kernel."""
    import torch

    B = len(lens)
    g = torch.Generator().manual_seed(B + max_pages)
    pages_per = [(l + P - 1) // P for l in lens]
    NB = sum(pages_per) + 8
    perm = torch.randperm(NB, generator=g)
    bt = torch.zeros(B, max_pages, dtype=torch.int32)
    c = 0
    for b, npg in enumerate(pages_per):
        bt[b, :npg] = perm[c:c + npg].int()
        c += npg
    cl = torch.tensor(lens, dtype=torch.int32)
    q = torch.randn(B, Hq, D, generator=g).half()
    kc = torch.empty(NB, Hkv * D // 16, P, 16, dtype=torch.float16)
    vc = torch.empty_like(kc)
    for i in range(0, NB, 64):
        kc[i:i + 64] = torch.randn(min(64, NB - i), Hkv * D // 16, P, 16, generator=g).half()
        vc[i:i + 64] = torch.randn(min(64, NB - i), Hkv * D // 16, P, 16, generator=g).half()
    sum_ctx = int(sum(lens))
    alg = sum_ctx * Hkv * D * 2 * 2 + 2 * B * Hq * D * 2 + bt.numel() * 4 + B * 4
    cache_bytes = 2 * kc.numel() * 2
    n = n_sets_for(cache_bytes, lo=2, hi=8)
    qd, btd, cld = q.to(dev), bt.to(dev), cl.to(dev)
    kcs = [kc.to(dev) for _ in range(n)]
    vcs = [vc.to(dev) for _ in range(n)]
    ws_bytes = L.lib.aops_paged_attention_workspace(B, Hq, Hkv, D, P, max_pages)
    wss = [torch.empty(ws_bytes, dtype=torch.uint8, device=dev) for _ in range(n)]
    outs = [torch.empty(B, Hq, D, dtype=torch.float16, device=dev) for _ in range(n)]

    def mk(i):
        return lambda: L.check(L.lib.aops_paged_attention_f16(
            qd.data_ptr(), kcs[i].data_ptr(), vcs[i].data_ptr(), btd.data_ptr(), cld.data_ptr(), outs[i].data_ptr(),
            wss[i].data_ptr(), ws_bytes, B, Hq, Hkv, D, P, max_pages, NB, L.stream()))

    med, mn = time_graph([mk(i) for i in range(n)], min_launches=64)
    cpu_ms = None
    if cpu:
        cpu_ms, ref = time_cpu(lambda: R.paged_attention_ref(q, kc, vc, bt, cl))
    else:
        ref = R.paged_attention_ref(q, kc, vc, bt, cl)
    torch.testing.assert_close(outs[-1].cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)
    e = entry("paged_attention", config, f"q [{B},{Hq},{D}], block {P}, table width {max_pages} pages, sum(context)={sum_ctx}",
              "hbm", alg, 0, med, mn, None, cpu_ms, torch.get_num_threads(), note)
    e["workspace_bytes"] = ws_bytes
    return e


def bench_pa_more(L, R, dev, cpu):
    import torch

    g = torch.Generator().manual_seed(11)
    ragged8 = torch.randint(512, 4097, (8,), generator=g).tolist()
    skew64 = [32768] + [128] * 63
    skew128 = [32768] + [128] * 127
    return [
        bench_pa_shape(L, R, dev, cpu, "5 at batch 8: contexts ~U[512,4096]", ragged8, 32, 8, 128, 128, 32,
                       "pa_decode_balanced (one equal share of the token stream per CU) + pa_decode_merge"),
        bench_pa_shape(L, R, dev, cpu, "5 at batch 1: one context of 32768 tokens", [32768], 32, 8, 128, 128, 256,
                       "pa_decode_balanced + pa_decode_merge"),
        bench_pa_shape(L, R, dev, cpu, "5 skewed: 64 sequences, one of 32768 tokens and 63 of 128", skew64, 32, 8, 128, 128, 256,
                       "pa_decode_balanced + pa_decode_merge (a block table that allows more than 4096 tokens)"),
        bench_pa_shape(L, R, dev, cpu, "5 skewed: 128 sequences, one of 32768 tokens and 127 of 128", skew128, 32, 8, 128, 128, 256,
                       "pa_decode_balanced (partition computed by every workgroup in LDS) + pa_decode_merge (more sequences than lanes)"),
        bench_pa_shape(L, R, dev, cpu, "5 with head_dim 96: 16 sequences of 2048 tokens", [2048] * 16, 16, 4, 96,
                       16, 128, "matrix-core kernel with three slices of 32 per head; balanced partition + merge"),
        bench_pa_shape(L, R, dev, cpu, "5 with head_dim 192: 64 sequences of 2048 tokens", [2048] * 64, 32, 8, 192,
                       128, 16, "matrix-core kernel with six slices; whole sequences per workgroup"),
        bench_pa_shape(L, R, dev, cpu, "5 with head_dim 80: 64 sequences of 2048 tokens", [2048] * 64, 32, 8, 80,
                       128, 16, "two slices of 32 and a half slice of 16 per head"),
        bench_pa_shape(L, R, dev, cpu, "5 with 32 query heads per kv head: 64 sequences of 2048 tokens", [2048] * 64, 256, 8,
                       128, 128, 16, "two sub-groups of 16 query heads per workgroup on one set of K/V registers"),
        bench_pa_shape(L, R, dev, cpu, "5 with 24-token pages (generic kernel): 16 sequences of 2048 tokens", [2048] * 16, 16, 4,
                       128, 24, 96, "pa_decode_generic: page sizes that are not a multiple of 16 tokens"),
    ]


def bench_dense(L, R, dev):
    """A compute-bound dense product through aops_matmul_nt_f16: HBM is out of the picture (805 MB against 1.1
    TFLOP), so the line isolates the k loop of the persistent kernel the MoE GEMMs run."""
    import torch

    m = k = n = 8192
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(m, k, generator=g)).half()
    w = (torch.randn(n, k, generator=g) / k ** 0.5).half()
    xd, wd = x.to(dev), w.to(dev)
    y = torch.empty(m, n, dtype=torch.float16, device=dev)
    call = lambda: L.check(L.lib.aops_matmul_nt_f16(xd.data_ptr(), wd.data_ptr(), y.data_ptr(), m, k, n, L.stream()))
    med, mn = time_graph([call], min_launches=32, trials=3)
    rows = torch.randint(0, m, (48,), generator=g)
    ref = x[rows].float() @ w.float().T
    torch.testing.assert_close(y[rows.to(dev)].cpu().float(), ref, rtol=2e-2, atol=2e-2)
    flops = 2 * m * k * n
    alg = (m * k + n * k + m * n) * 2
    e = entry("matmul", "dense 8192 x 8192 x 8192 (compute bound; not a BASELINE config)", f"x [{m},{k}] @ w [{n},{k}]^T f16",
              "mfma", alg, flops, med, mn, None, None, 1,
              "the persistent 320 x 256 kernel on one group; checked against the fp32 product on 48 sampled rows")
    return e


def bench_gmm_probe(L, R, dev, only=None):
    """Where the time of the MoE GEMMs goes, from kernels in the library alone: the persistent grouped-matmul kernel
    on configs[3] with parts of its k loop switched off (aops_grouped_matmul_probe_f16), and a pure read stream
    with the access pattern of its weight copies next to a linear stream of the same bytes
    (aops_probe_read_stream).  Results of the switched-off forms are wrong by construction; only times count."""
    import torch

    E, hidden, inter, tokens, topk = 128, 2048, 768, 4096, 8
    rows = tokens * topk
    torch.manual_seed(0)
    gl = R.make_group_list(torch.randint(0, E, (rows,)), E).to(dev)
    out = []
    gl_moe, rows_moe = gl, rows
    for which, K, N in (("gate_up", hidden, 2 * inter), ("down", inter, hidden), ("dense", 8192, 8192)):
        if only and which != only:   # one shape alone, so that a counter pass has one shape per kernel name
            continue
        g = torch.Generator(device=dev).manual_seed(1)
        moe = which != "dense"   # the dense product: one group of 8192 rows (320-row tiles here, 256-row tiles in the "dense" line)
        E, rows = (128, rows_moe) if moe else (1, 8192)
        gl = gl_moe if moe else torch.tensor([rows], dtype=torch.int64, device=dev)
        sets = 2 if moe else 1
        xs = [torch.randn(rows, K, generator=g, device=dev, dtype=torch.float16) for _ in range(sets)]
        ws = [torch.randn(E, N, K, generator=g, device=dev, dtype=torch.float16) * 0.02 for _ in range(sets)]
        ys = [torch.empty(rows, N, device=dev, dtype=torch.float16) for _ in range(sets)]
        flops = 2 * rows * K * N
        alg = rows * K * 2 + E * N * K * 2 + rows * N * 2 + E * 8

        def timed(parts_off, wsrc=None, ld=None):
            if parts_off == 0:
                calls = [(lambda i=i: L.check(L.lib.aops_grouped_matmul_variant_f16(
                    6, xs[i].data_ptr(), ws[i].data_ptr(), gl.data_ptr(), ys[i].data_ptr(), rows, K, E, N, L.stream())))
                    for i in range(sets)]
            else:
                calls = [(lambda i=i: L.check(L.lib.aops_grouped_matmul_probe_f16(
                    parts_off, xs[i].data_ptr(), (wsrc or ws)[i].data_ptr(), ld or K, gl.data_ptr(), ys[i].data_ptr(), rows, K,
                    E, N, L.stream()))) for i in range(sets)]
            return time_graph(calls, min_launches=40, trials=3)

        for parts_off, what in ((0, "whole kernel"), (9, "operand copies and barriers only"), (11, "weight copies only"),
                                (13, "activation copies only"), (6, "MFMAs and LDS fragment reads only"), (14, "MFMAs only"),
                                (1, "copies and LDS fragment reads, no MFMAs"), (8, "copies and MFMAs, no LDS fragment reads"),
                                (25, "operand copies and barriers only, weights in 256-byte pieces from half the rows per tile"),
                                (27, "weight copies only, in 256-byte pieces from half the rows per tile")):
            med, mn = timed(parts_off)
            # the whole kernel goes through the library's own choice of tile height (256 rows for the dense product)
            label = f"probe 4: MoE {which}" if moe else f"probe dense 8192^3 ({256 if parts_off == 0 else 320}-row tiles)"
            e = entry("grouped_matmul_probe", f"{label}, {what}", f"x [{rows},{K}] @ w [{E},{K},{N}] f16",
                      "mfma", alg, flops, med, mn, None, None, 1,
                      None if parts_off == 0 else "parts of the k loop switched off: results wrong by construction, time only")
            e["parts_off"] = parts_off
            out.append(e)
        # the same launch on operands that are all zero: the matrix cores' multipliers do not switch, the chip
        # stays inside its power limit at full clock, and what is left is the time of the operand copies
        for i in range(sets):
            xs[i].zero_()
            ws[i].zero_()
        med, mn = timed(0)
        label = f"probe 4: MoE {which}" if moe else "probe dense 8192^3 (256-row tiles)"
        out.append(entry("grouped_matmul_probe", f"{label}, whole kernel on all-zero operands",
                         f"x [{rows},{K}] @ w [{E},{K},{N}] f16", "mfma", alg, flops, med, mn, None, None, 1,
                         "the same launch as the whole-kernel line, correct results (zeros); the difference to that line "
                         "is what the power limit costs with operands that change"))
        if not moe:
            del xs, ws, ys
            torch.cuda.empty_cache()
            continue
        g = torch.Generator(device=dev).manual_seed(1)   # back to the operands of the lines above
        xs = [torch.randn(rows, K, generator=g, device=dev, dtype=torch.float16) for _ in range(sets)]
        ws = [torch.randn(E, N, K, generator=g, device=dev, dtype=torch.float16) * 0.02 for _ in range(sets)]
        # the same GEMM on weights whose rows are padded by one cache line (aops_grouped_matmul_ldw_f16): what the
        # power-of-two row stride of the reference's layout costs
        ldw = K + 64
        wps = []
        for i in range(sets):
            wp = torch.zeros(E, N, ldw, device=dev, dtype=torch.float16)
            wp[:, :, :K] = ws[i]
            wps.append(wp)
        y_pad = torch.empty(rows, N, device=dev, dtype=torch.float16)
        L.check(L.lib.aops_grouped_matmul_ldw_f16(xs[0].data_ptr(), wps[0].data_ptr(), ldw, gl.data_ptr(), y_pad.data_ptr(),
                                                  rows, K, E, N, L.stream()))
        L.check(L.lib.aops_grouped_matmul_variant_f16(6, xs[0].data_ptr(), ws[0].data_ptr(), gl.data_ptr(), ys[0].data_ptr(),
                                                      rows, K, E, N, L.stream()))
        assert torch.equal(y_pad, ys[0]), "padded weight rows must give the same bits"
        calls = [(lambda i=i: L.check(L.lib.aops_grouped_matmul_ldw_f16(
            xs[i].data_ptr(), wps[i].data_ptr(), ldw, gl.data_ptr(), ys[i].data_ptr(), rows, K, E, N, L.stream())))
            for i in range(sets)]
        med, mn = time_graph(calls, min_launches=40, trials=3)
        out.append(entry("grouped_matmul_ldw", f"probe 4: MoE {which}, weight rows padded to {2 * ldw} bytes (extension)",
                         f"x [{rows},{K}] @ w [{E},{K},{N}] f16, row stride {ldw}", "mfma", alg, flops, med, mn, None, None, 1,
                         "same kernel and same bits as the whole-kernel line; the caller pads the static weights once"))
        for parts_off, what in ((9, "operand copies and barriers only"), (11, "weight copies only"),
                                (25, "operand copies and barriers only, weights in 256-byte pieces"),
                                (27, "weight copies only, in 256-byte pieces")):
            med, mn = timed(parts_off, wps, ldw)
            e = entry("grouped_matmul_probe", f"probe 4: MoE {which}, weight rows padded to {2 * ldw} bytes, {what}",
                      f"x [{rows},{K}] @ w [{E},{K},{N}] f16, row stride {ldw}", "mfma", alg, flops, med, mn, None, None, 1,
                      "parts of the k loop switched off: results wrong by construction, time only")
            e["parts_off"] = parts_off
            out.append(e)
        del wps, y_pad
        # the weight bytes of this GEMM as a pure read stream: the kernel's pattern, longer pieces, and linear
        wbytes = E * N * K * 2
        sink = torch.zeros(1, dtype=torch.float32, device=dev)
        for seg, row_bytes, via_lds, what in (
                (128, 2 * K, 0, f"128-byte pieces one weight row ({2 * K} B) apart, as the kernel copies them"),
                (256, 2 * K, 0, "256-byte pieces one weight row apart"),
                (512, 2 * K, 0, "512-byte pieces one weight row apart"),
                (128, 2 * K + 128, 0, f"128-byte pieces {2 * K + 128} B apart (what a row padded by one line would give)"),
                (1024, 1024, 0, "the same bytes read linearly (1 KiB per row of the probe)"),
                (128, 2 * K, 1, f"128-byte pieces {2 * K} B apart, copied straight into LDS (the kernel's copy instruction)"),
                (128, 2 * K + 128, 1, f"128-byte pieces {2 * K + 128} B apart, copied straight into LDS"),
                (1024, 1024, 1, "read linearly, copied straight into LDS")):
            if row_bytes % seg != 0:
                continue
            nrows = wbytes // row_bytes // 128 * 128
            calls = [(lambda i=i: L.check(L.lib.aops_probe_read_stream(ws[i].data_ptr(), nrows, row_bytes, seg, via_lds,
                                                                        sink.data_ptr(), L.stream()))) for i in range(sets)]
            med, mn = time_graph(calls, min_launches=40, trials=3)
            out.append(entry("read_stream_probe", f"probe 4: weights of MoE {which} as a read stream, {what}",
                             f"[{nrows},{row_bytes}] bytes, 128 rows per workgroup", "hbm", nrows * row_bytes, 0, med, mn,
                             None, None, 1))
        del xs, ws, ys
        torch.cuda.empty_cache()
    if only is None:
        # what the matrix cores sustain by themselves: fp16 MFMAs of the two shapes on operands in registers
        sink = torch.zeros(1, dtype=torch.float32, device=dev)
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        iters = 8192
        flops = cus * 8 * iters * 8 * 32768
        gen = torch.Generator(device=dev).manual_seed(3)
        for data, operands in (("all-zero operands", torch.zeros(16 * 64 * 8, device=dev, dtype=torch.float16)),
                               ("operands uniform in [-2, 2)", (torch.rand(16 * 64 * 8, generator=gen, device=dev) * 4 - 2).half())):
            for shape, name in ((32, "v_mfma_f32_32x32x16_f16"), (16, "v_mfma_f32_16x16x32_f16")):
                calls = [lambda: L.check(L.lib.aops_probe_mfma_rate(shape, operands.data_ptr(), iters, sink.data_ptr(), L.stream()))]
                med, mn = time_graph(calls, min_launches=6, trials=3)
                out.append(entry("mfma_rate_probe", f"probe: {name} alone, {data}", f"{cus} CUs x 8 waves x {iters} rounds",
                                 "mfma", 16384 * cus * 8, flops, med, mn, None, None, 1,
                                 "MFMAs on registers, nothing else: the rate the matrix cores sustain for this operand content"))

    return out


def kernel_source_digest():
    """Digest of the paged-attention kernels' source: the recorded HBM-traffic figure names the digest it was
    measured on and is dropped when the source has changed since."""
    h = hashlib.sha256()
    for name in ("paged_attention.hip", "aops_common.h"):
        with open(os.path.join(ROOT, "ascend-ops_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


PER_KERNEL_FIELDS = ["op", "config", "us", "frac_of_peak", "bound", "launch_floor_us", "cpu_ms"]
_SHORT = {"grouped_matmul": "gmm", "grouped_matmul_swiglu": "gmm+swiglu", "grouped_matmul_swiglu_gather": "gmm+swiglu+gather",
          "paged_attention": "pa", "reshape_and_cache": "cache", "add_rms_norm": "norm"}


def compact(e):
    """One per_kernel row of the headline, in the order of PER_KERNEL_FIELDS (a list keeps the line short)."""
    if "error" in e:
        return [e.get("op_group"), "error: " + e["error"][:60]]
    frac = e.get("mfma_frac") if e.get("bound") == "mfma" else e.get("hbm_frac")
    cfg = e["config"]
    for cut in (" (", ": add", ": resh", ": rope", ": MLP"):
        cfg = cfg.split(cut)[0]
    cpu = e.get("cpu_ms")
    return [_SHORT.get(e["op"], e["op"]), cfg[:34], round(e["gpu_us"], 1), None if frac is None else round(frac, 3),
            e.get("bound"), e.get("launch_floor_us"), None if cpu is None else round(cpu, 1)]


# --------------------------------------------------------------------------------------- main
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--ops", default="all", help="comma list of: pa,norm,cache,mlp,moe,rope,scaled or all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--skip-headline", action="store_true",
                    help="profiler runs of single operators: do not run the paged-attention headline workload "
                         "(the last line then carries the per-operator records only)")
    ap.add_argument("--calib", action="store_true",
                    help="also run a plain elementwise copy of 512 MiB (reads 512 MiB, writes 512 MiB): the known-size "
                         "kernel against which FETCH_SIZE / WRITE_SIZE counters of a profiler run are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (every operator is independent per token, per "
                 "(sequence, kv head) or per expert and shards without an internal exchange); use --gpus 1")

    import torch

    import __graft_entry__ as entry_points
    entry_points._build_if_absent()          # a fresh checkout holds no built library
    import ascend910a_extras.ops as ops      # the product; raises if libaops.so is missing
    import oracle.ops_ref as R               # checker + timed CPU baseline only

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = Lib()
    cpu = not args.no_cpu
    want = set(args.ops.split(","))
    allops = "all" in want
    cores = torch.get_num_threads()
    log(f"[bench] device: {torch.cuda.get_device_name(0)}; host threads: {cores} (os.cpu_count()={os.cpu_count()})")
    log(f"[bench] denominators: HBM {HBM_PEAK_GBPS} GB/s, fp16 MFMA {MFMA_F16_PEAK_TFLOPS} TFLOP/s")

    per_op = []

    def run(tag, fn):
        if allops or tag in want:
            t0 = time.perf_counter()
            try:
                res = fn()
            except Exception as exc:  # the headline line must still be printed; the failure goes into it
                log(f"[bench] {tag} FAILED: {exc!r}")
                res = {"op_group": tag, "error": repr(exc)[:400]}
                torch.cuda.synchronize()
            res = res if isinstance(res, list) else [res]
            per_op.extend(res)
            for r in res:
                log(f"[bench] {json.dumps(r)}")
            log(f"[bench] {tag} done in {time.perf_counter() - t0:.1f}s")
            torch.cuda.empty_cache()

    if args.skip_headline:
        for tag, fn in (("moe_gate_up", lambda: bench_moe_one(L, ops, R, dev, "gate_up")),
                        ("moe_down", lambda: bench_moe_one(L, ops, R, dev, "down")),
                        ("moe_gate_up_padded", lambda: bench_moe_one(L, ops, R, dev, "gate_up_padded")),
                        ("dense", lambda: bench_dense(L, R, dev)),
                        ("gmm_probe", lambda: bench_gmm_probe(L, R, dev)),
                        ("gmm_probe_gate_up", lambda: bench_gmm_probe(L, R, dev, "gate_up")),
                        ("gmm_probe_down", lambda: bench_gmm_probe(L, R, dev, "down")),
                        ("gmm_probe_dense", lambda: bench_gmm_probe(L, R, dev, "dense")),
                        ("pa_more", lambda: bench_pa_more(L, R, dev, cpu))):
            if tag in want:
                run(tag, fn)
        print(json.dumps({"per_op": per_op}), flush=True)
        return

    # ------------------------------------------------------------------ primary: paged attention
    t0 = time.perf_counter()
    wl = PagedAttentionWorkload(R, dev)
    log(f"[bench] config 5 inputs ready in {time.perf_counter() - t0:.1f}s; sum(context)={wl.sum_ctx}")
    for i in range(args.warmup):
        wl.step(ops, i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        wl.step(ops, i)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    pa = bench_paged_attention(L, ops, R, dev, cpu, wl)
    log(f"[bench] {json.dumps(pa)}")
    per_op.append(pa)
    sum_ctx, alg_bytes = wl.sum_ctx, wl.alg_bytes
    del wl
    torch.cuda.empty_cache()

    run("norm", lambda: bench_add_rms_norm(L, ops, R, dev, cpu, 128, "1: add_rms_norm", floor=True))
    run("cache", lambda: bench_reshape_and_cache(L, ops, R, dev, cpu, 2048, "2: reshape_and_cache", floor=True))
    run("rope", lambda: bench_rope(L, ops, R, dev, cpu, 64, "5: rope", floor=True))
    run("mlp", lambda: bench_mlp(L, ops, R, dev, cpu))
    run("moe", lambda: bench_moe(L, ops, R, dev, cpu))
    if "moe_gate_up" in want:
        run("moe_gate_up", lambda: bench_moe_one(L, ops, R, dev, "gate_up"))
    if "moe_down" in want:
        run("moe_down", lambda: bench_moe_one(L, ops, R, dev, "down"))
    run("pa_more", lambda: bench_pa_more(L, R, dev, cpu))
    run("dense", lambda: bench_dense(L, R, dev))
    run("gmm_probe", lambda: bench_gmm_probe(L, R, dev))
    run("scaled", lambda: [
        bench_add_rms_norm(L, ops, R, dev, False, 16384, "1 scaled x128: add_rms_norm",
                           "scaled shape: shows the kernel's asymptotic bandwidth, not a BASELINE config"),
        bench_reshape_and_cache(L, ops, R, dev, False, 65536, "2 scaled x32: reshape_and_cache",
                                "scaled shape: shows the kernel's asymptotic bandwidth, not a BASELINE config"),
        bench_reshape_and_cache(L, ops, R, dev, False, 65536, "2 scaled x32, slots in page order: reshape_and_cache",
                                "scaled shape with the slot pattern of a prefill (whole pages in token order, pages "
                                "scattered) instead of BASELINE's random permutation", consecutive=True),
        bench_swiglu(L, ops, R, dev, False, 8192, 14336, "3 scaled x32: swiglu",
                     "scaled shape: shows the kernel's asymptotic bandwidth, not a BASELINE config"),
        bench_rope(L, ops, R, dev, False, 16384, "5 scaled x256: rope",
                   "scaled shape: shows the kernel's asymptotic bandwidth, not a BASELINE config"),
    ])

    if args.calib:
        src = torch.ones(256 << 20, dtype=torch.float16, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)  # one vectorized elementwise kernel: 512 MiB in, 512 MiB out
        torch.cuda.synchronize()
        log("[bench] calibration copy done: 3 launches, 536870912 B read + 536870912 B written each")
        del src, dst

    # HBM bytes per launch measured with rocprofv3 counters: a recorded summary that names the digest of the kernel
    # source it was measured on; a figure measured on other source is dropped (null) rather than reported stale
    traffic, traffic_note = None, None
    tfile = os.path.join(ROOT, "profiles", "pa_decode_config5_hbm_traffic.txt")
    if os.path.exists(tfile):
        recorded, digest = None, None
        for ln in open(tfile):
            if ln.strip().startswith("traffic_bytes_per_launch:"):
                recorded = int(ln.split(":")[1])
            if ln.strip().startswith("kernel_source_digest:"):
                digest = ln.split(":")[1].strip()
        if recorded is not None and digest == kernel_source_digest():
            traffic = recorded
            traffic_note = ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known size; recorded in "
                            "profiles/pa_decode_config5_hbm_traffic.txt for this kernel source")
        else:
            traffic_note = "recorded figure was measured on other kernel source (digest mismatch): dropped"

    # the full per-operator records on their own line, BEFORE the headline (which must be the last line)
    print(json.dumps({"per_op": per_op}), flush=True)

    wanted = ("1:", "2:", "3: MLP swiglu", "5: rope", "4: MoE gate_up", "4: MoE down", "5 at batch 8", "5 at batch 1",
              "5 skewed: 64", "5 with head_dim 96", "dense 8192")
    unwanted = ("4: MoE gate_up + down", "4: MoE gate_up + activation + row gather")
    per_kernel = [compact(e) for e in per_op
                  if "error" in e or (any(e.get("config", "").startswith(w) for w in wanted)
                                      and not any(e.get("config", "").startswith(u) for u in unwanted))]
    if traffic_note and traffic is None:
        log(f"[bench] roofline.traffic: {traffic_note}")
    def find(prefix):
        return next((e for e in per_op if e.get("config", "").startswith(prefix)), None)

    gmm_sum = find("4: MoE gate_up + down")
    gmm_up = next((e for e in per_op if e.get("config") == "4: MoE gate_up"), None)
    gmm_down = next((e for e in per_op if e.get("config") == "4: MoE down"), None)
    gmm_cpu = [e.get("cpu_ms") for e in (gmm_up, gmm_down) if e]
    # flat scalar copies of the per-operator fractions: a reader that keeps only scalar keys of `roofline` still
    # sees the GEMM half of the metric and the four small operators next to the paged-attention figure
    flat = {}
    if gmm_sum:
        flat.update(gmm_frac=gmm_sum["mfma_frac"], gmm_tflops=gmm_sum["TFLOPs"], gmm_us=round(gmm_sum["gpu_us"], 1),
                    gmm_kernel="grouped_matmul_persistent_kernel<5,2,4,false,false> (gate_up + down of configs[3])")
    for key, e in (("gmm_gate_up", gmm_up), ("gmm_down", gmm_down)):
        if e and "mfma_frac" in e:
            flat[key + "_frac"] = e["mfma_frac"]
            flat[key + "_us"] = round(e["gpu_us"], 1)
            flat[key + "_frac_of_hbm_ceiling"] = e.get("frac_of_roofline_ceiling")
    for key, prefix in (("add_rms_norm", "1: add_rms_norm"), ("reshape_and_cache", "2: reshape_and_cache"),
                        ("swiglu", "3: MLP swiglu"), ("rope", "5: rope"), ("swiglu_moe", "4: MoE activation"),
                        ("add_rms_norm_scaled", "1 scaled"), ("reshape_and_cache_scaled", "2 scaled x32: resh"),
                        ("swiglu_scaled", "3 scaled"), ("rope_scaled", "5 scaled"),
                        ("pa_batch8", "5 at batch 8"), ("pa_batch1", "5 at batch 1"), ("pa_skewed64", "5 skewed: 64"),
                        ("pa_skewed128", "5 skewed: 128"), ("pa_head_dim96", "5 with head_dim 96")):
        e = find(prefix)
        if e and "hbm_frac" in e:
            flat[key + "_frac"] = e["hbm_frac"]
            flat[key + "_us"] = round(e["gpu_us"], 2)
    gbps_wall = alg_bytes / (ms_per_step * 1e-3) / 1e9
    gbps_kernel = alg_bytes / (pa["gpu_us"] * 1e-6) / 1e9
    line = {
        "metric": "GB/s & % HBM roofline (norm/cache/PA); GMM TFLOPS & % fp16 MFMA peak",
        "value": round(gbps_wall, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[4]: paged-attention decode, B=64, 32q/8kv heads, D=128, block 128, ctx~U[512,4096]",
            "sum_context_tokens": sum_ctx,
            "algorithmic_bytes_per_step": alg_bytes,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbps_kernel, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(gbps_kernel / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "kernel": "pa_decode_partial<128,1>",
            "us_per_call": pa["gpu_us"],
            **flat,
            "gmm": None if not gmm_sum else {
                "config": "configs[3] gate_up+down", "bound": "mfma", "TFLOPs": gmm_sum["TFLOPs"],
                "peak": MFMA_F16_PEAK_TFLOPS, "frac": gmm_sum["mfma_frac"], "us": round(gmm_sum["gpu_us"], 1),
                "cpu_ms": None if not all(gmm_cpu) or len(gmm_cpu) != 2 else round(sum(gmm_cpu), 1),
            },
            "per_kernel_fields": PER_KERNEL_FIELDS,
            "per_kernel": per_kernel,
        },
        "cpu_baseline": None if not cpu else {
            "value": round(alg_bytes / (pa["cpu_ms"] * 1e-3) / 1e9, 3),
            "unit": "GB/s",
            "cores": cores,
            "kind": "port",
            "sample": "full configs[4] batch; torch fp32 oracle",
            "runs": f"1 warm-up + median of {CPU_RUNS}",
            "ms": pa["cpu_ms"],
            "gmm_ms": None if not all(gmm_cpu) or len(gmm_cpu) != 2 else round(sum(gmm_cpu), 1),
        },
    }
    print(json.dumps(line, separators=(",", ":")), flush=True)


if __name__ == "__main__":
    main()
