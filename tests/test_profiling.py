"""The chrome-trace helper (counterpart of prof() in the reference's benchmark/test_graph.py:15-53)."""
import json

import pytest
import torch


def test_prof_writes_a_chrome_trace_without_a_gpu(tmp_path):
    import ascend910a_extras.profiling as profiling

    calls = []
    x = torch.randn(64, 64)
    path = str(tmp_path / "trace.json")
    profiling.prof(lambda: calls.append((x @ x).sum()), path, iter_num=3)
    assert len(calls) == 3
    events = json.load(open(path))["traceEvents"]
    assert any("mm" in ev.get("name", "") for ev in events)
    with pytest.raises(ValueError):
        profiling.prof(lambda: None, path, iter_num=1)


@pytest.mark.gpu
def test_prof_records_the_library_kernels(ops, dev, tmp_path):
    import ascend910a_extras.profiling as profiling

    x = torch.randn(128, 4096, dtype=torch.float16, device=dev)
    w = torch.ones(4096, dtype=torch.float16, device=dev)
    path = str(tmp_path / "trace.json")
    profiling.prof(lambda: ops.add_rms_norm(x, x, w, 1e-6), path, iter_num=4)
    times = profiling.kernel_times(path)
    hits = {name: t for name, t in times.items() if "add_rms_norm" in name}
    assert hits, f"no add_rms_norm kernel in the trace: {list(times)}"
    assert sum(len(t) for t in hits.values()) == 3          # the first of four calls is skipped
    assert all(0 < d < 1000 for t in hits.values() for d in t)
