"""Chrome-trace helper for the operators: the counterpart of ``prof(fn, trace_fn)`` in the reference's
``benchmark/test_graph.py:15-53``, on ``torch.profiler`` instead of ``torch_npu.profiler``.

``prof(fn, "trace.json")`` calls ``fn`` a few times, records host activity and (on a GPU) every kernel the
calls enqueue, and writes a trace that ``chrome://tracing`` or Perfetto opens.  The first call is skipped
as warm-up, as in the reference (``skip_first=1``).  ``kernel_times`` reads the kernel durations back out
of such a trace."""
from __future__ import annotations

import json
from typing import Callable, Dict, List

import torch


def prof(fn: Callable[[], object], trace_fn: str, iter_num: int = 4, with_stack: bool = False) -> None:
    """Runs ``fn`` ``iter_num`` times (the first untraced) and exports a chrome trace to ``trace_fn``."""
    if iter_num < 2:
        raise ValueError("prof: iter_num must be at least 2 (one skipped call, one traced)")
    on_gpu = torch.cuda.is_available()
    activities = [torch.profiler.ProfilerActivity.CPU]
    if on_gpu:
        activities.append(torch.profiler.ProfilerActivity.CUDA)
    with torch.profiler.profile(
        activities=activities,
        schedule=torch.profiler.schedule(wait=0, warmup=0, active=iter_num - 1, repeat=1, skip_first=1),
        record_shapes=False,
        profile_memory=False,
        with_stack=with_stack,
    ) as profiler:
        for _ in range(iter_num):
            fn()
            if on_gpu:
                torch.cuda.synchronize()
            profiler.step()
    profiler.export_chrome_trace(trace_fn)


def kernel_times(trace_fn: str) -> Dict[str, List[float]]:
    """Durations in microseconds of the GPU kernels in a trace written by ``prof``, by kernel name."""
    with open(trace_fn) as f:
        events = json.load(f).get("traceEvents", [])
    out: Dict[str, List[float]] = {}
    for ev in events:
        if ev.get("cat") == "kernel" and "dur" in ev:
            out.setdefault(ev["name"], []).append(float(ev["dur"]))
    return out
