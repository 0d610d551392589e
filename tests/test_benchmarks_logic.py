"""The benchmark harness (exact_amd/benchmarks.py) run end to end at a tiny
scale on the emulated backend: graph generator, epoch loop, the extra kernel
measurements and the byte formulas -- so that the code bench.py runs on the
GPU box has executed at least once before it gets there."""
import time

import numpy as np
import pytest
import torch

from exact_amd import benchmarks as bm


@pytest.fixture
def cpu_harness(backend, monkeypatch):
    if backend.type != "cpu":
        pytest.skip("logic test of the harness; the GPU runs it through bench.py")

    def wall_time(fn, reps=1, warm=0):
        for _ in range(warm):
            fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    def wall_launch_times(fn, reps=2, warm=0):
        t = wall_time(lambda: fn(0), reps=2) * 1e6
        return t, t

    monkeypatch.setattr(bm, "event_time", wall_time)
    monkeypatch.setattr(bm, "launch_times", wall_launch_times)
    monkeypatch.setattr(bm, "_sync", lambda: None)
    monkeypatch.setattr(bm, "_reset_peak", lambda d: None)
    monkeypatch.setattr(bm, "_peak_gb", lambda d: 0.0)
    monkeypatch.setattr(bm, "_trim", lambda: None)
    monkeypatch.setattr(bm, "bench_device", lambda: backend)
    return backend


def test_powerlaw_graph_is_symmetric_simple_and_heavy_tailed(cpu_harness):
    adj = bm.powerlaw_graph(5000, 30000, seed=1, device=cpu_harness)
    rowptr, col, value = adj.csr()
    assert value is None and rowptr[-1].item() == col.numel()
    row = adj.storage.row()
    assert (row != col).all()                                    # no self loops
    key = row * 5000 + col
    assert key.unique().numel() == key.numel()                   # no duplicates
    assert set((col * 5000 + row).tolist()) == set(key.tolist())  # symmetric
    deg = (rowptr[1:] - rowptr[:-1]).float()
    assert 40000 < col.numel() < 70000 and deg.max() > 8 * deg.mean()
    assert (torch.sort(key).values == key).all()                 # CSR order


def test_byte_formulas():
    # config 3, K = 256: 378.0 MB with int64 indices and values (published denominator)
    b = bm.spmm_bytes(169343, 169343, 2_480_000, 256, 8, True)
    assert abs(b / 1e6 - 378.0) < 1.0


def test_harness_runs_every_part_at_tiny_scale(cpu_harness):
    x = torch.randn(65, 64, device=cpu_harness)
    logs = []
    out = bm.run(x, logs.append, scale=0.0005, epochs=1, warmup=0)
    assert "error" not in out["kernels"], out["kernels"]
    for name in ("relu_fwd", "relu_bwd", "dropout_fwd", "dropout_bwd", "relu_dropout_fwd", "rp_fwd", "rp_bwd", "rp_compress_int2",
                 "rp_decompress_int2"):
        assert out["kernels"][name]["us"] > 0
    for name in bm.EPOCH_CONFIGS:
        assert "error" not in out[name] and "skipped" not in out[name], (name, out[name])
        assert out[name]["epochs_per_s"] > 0 and np.isfinite(out[name]["last_loss"])
        assert out[name]["spmm"]["fwd_us"] > 0
    assert out["cfg5_sage_int1_rp0.25"]["bits"] == 1 and out["cfg3_gcn_int2"]["index_dtype"] == "int32"


def test_bench_py_emits_the_contract_line(cpu_harness, capsys):
    """bench.py end to end (tiny rows, emulated kernels): one JSON line with
    the contract's keys, the roofline and the cpu_baseline objects."""
    import importlib
    import json
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    bench = importlib.import_module("bench")
    import bench as b2
    b2.cpu_baseline.__defaults__ = (0.2, 1)
    bench.main(["--rows", "203", "--steps", "2", "--warmup", "1", "--extras-scale", "0.0005", "--extras-in-process"])
    lines = [l for l in capsys.readouterr().out.splitlines() if l.strip()]
    assert len(lines) == 1
    r = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in r, key
    assert r["unit"] == "GB/s" and r["n_gpus"] == 1 and r["vs_baseline"] is None and "workload" in r["config"]
    assert set(r["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"} and r["roofline"]["peak"] == 8000.0
    assert set(r["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"} and r["cpu_baseline"]["kind"] == "port"
    assert len(r["kernels"]) == 12 and set(r["epochs_per_s"]) == set(bm.EPOCH_CONFIGS)
    assert sum("supplied noise" in k["kernel"] for k in r["kernels"]) == 4          # the parity mode beside the headline
    assert r["roofline"]["traffic_probe"]["us"] > 0                                  # the same traffic without arithmetic, timed beside it
    assert sum("frac_of_traffic_probe" in k for k in r["kernels"]) == 4
    assert r["single_buffer_set"]["value"] > 0 and r["config"]["buffer_sets"] == 4
    for name in bm.EPOCH_CONFIGS:
        assert 0 < r["epoch_roofline"][name]["frac"] and r["epoch_roofline"][name]["algo_bytes_per_epoch"] > 0
    with pytest.raises(SystemExit):
        bench.main(["--gpus", "2"])


def test_extras_entry_point_prints_one_json_line(cpu_harness, capsys, monkeypatch):
    """`python -m exact_amd.benchmarks extras` (the child bench.py starts)."""
    import json
    monkeypatch.setattr(bm, "run", lambda x, log, budget_s, scale: {"rows": x.shape[0], "scale": scale, "b": budget_s})
    bm._profile_target(["extras", "--rows", "65", "--cols", "64", "--scale", "0.5", "--budget", "3"])
    lines = [l for l in capsys.readouterr().out.splitlines() if l.strip()]
    assert len(lines) == 1 and json.loads(lines[0]) == {"rows": 65, "scale": 0.5, "b": 3.0}


def test_failed_extras_child_leaves_an_error_entry(monkeypatch):
    import os
    import subprocess
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench

    class Done:
        returncode, stdout = -6, "progress\n"
    monkeypatch.setattr(subprocess, "run", lambda *a, **k: Done())
    assert "exited with -6" in bench.run_extras(10, 8, 1.0)["error"]
    Done.returncode, Done.stdout = 0, 'noise\n{"kernels": {}}\n'
    assert bench.run_extras(10, 8, 1.0) == {"kernels": {}}

    def boom(*a, **k):
        raise subprocess.TimeoutExpired(a[0], 1)
    monkeypatch.setattr(subprocess, "run", boom)
    assert "exceeded" in bench.run_extras(10, 8, 1.0)["error"]


def test_epoch_entry_point(cpu_harness, capsys):
    """`python -m exact_amd.benchmarks epoch` (the target of a kernel trace of one model configuration)."""
    import json
    bm._profile_target(["epoch", "--config", "cfg3_gcn_int2", "--epochs", "1", "--warmup", "0", "--scale", "0.0005"])
    res = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert res["epochs_per_s"] > 0 and res["bits"] == 2


@pytest.mark.parametrize("kernel", ["pack", "unpack", "relu", "dropout", "relu_dropout_pack", "bn_relu_dropout_pack",
                                    "rp_fwd", "rp_bwd", "rp_pack", "copy"])
def test_kernel_trace_targets_run(cpu_harness, capsys, kernel):
    """`python -m exact_amd.benchmarks <kernel>`: every target launches its entry point with valid arguments."""
    bm._profile_target([kernel, "--rows", "70", "--cols", "64", "--reps", "2"])
    assert f"{kernel}: 2 launches on [70, 64] done" in capsys.readouterr().out
