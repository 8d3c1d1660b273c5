"""The benchmark's command-line contract on a machine without a GPU: it refuses more than one GPU with
a message, and without a GPU it stops with an error instead of printing a figure from some other path."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + list(args), stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = _bench("--gpus", "2")
    assert proc.returncode != 0
    assert b"ONE GPU" in proc.stderr and b"--gpus 2" in proc.stderr
    assert not proc.stdout.strip()


def test_no_gpu_means_no_number():
    from nvshmem_amd import hip
    try:
        has_gpu = hip.device_count() > 0
    except Exception:
        has_gpu = False
    if has_gpu:
        pytest.skip("a GPU is visible here")
    proc = _bench("--steps", "2", "--warmup", "1")
    assert proc.returncode != 0
    assert b"no GPU" in proc.stderr
    assert b"{" not in proc.stdout


def _fake_results(workloads):
    """Records of the shape bench.summarise() returns, for every workload name the benchmark has, with the
    longest values the real ones reach."""
    names = []
    for g in workloads.all_groups((None, None, None, __import__("numpy").array([1]))):
        names += g.names()
    rec = {"GBs": 12345.6, "frac_of_hbm_peak": 0.7512, "ms_per_step": 123.45678, "kernel_ms": 123.45678,
           "kernel_GBs": 12345.6, "kernel_frac_of_hbm_peak": 0.7512, "cache_resident": False,
           "algorithmic_bytes": 15032385536, "traffic": 15082734491, "dtype": "bf16", "verified": True,
           "config": {"npes": 8, "bytes_per_pe": 268435456, "blocks_per_pe": 16, "threads_per_block": 1024,
                      "is_get": 0, "payload_only_GBs": 12345.6, "note": "n" * 300, "workload": "w" * 400},
           "kernel": "k" * 120,
           "cpu_baseline": {"value": 320.09, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "s" * 120,
                            "single_thread": 21.8},
           "steps": 20}
    out = {n: dict(rec) for n in names}
    return out


def test_result_line_is_short_and_round_trips():
    """The result line must fit the bounded tail of stdout that the harness reads back, for every workload
    the benchmark has and with values of realistic worst-case length."""
    import json
    sys.path.insert(0, ROOT)
    import bench
    from nvshmem_amd import workloads
    results = _fake_results(workloads)
    assert len(results) >= 30 and workloads.HEADLINE in results
    cached = next(n for n in results if n != workloads.HEADLINE)
    results[cached].update(cache_resident=True, frac_of_hbm_peak=None, kernel_frac_of_hbm_peak=None)
    line = bench.result_line(results, workloads.HEADLINE, 5)
    text = json.dumps(line, separators=(",", ":"))
    assert len(text) < bench.MAX_LINE_BYTES and "\n" not in text
    back = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "verified"):
        assert key in back
    assert back["config"]["workload"] and back["n_gpus"] == 1
    assert set(back["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"}
    assert set(back["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"}
    assert set(back["workloads"]) == set(results)
    assert back["workloads"][cached][1] is None          # no HBM fraction for a cache-resident working set
    results[cached]["verified"] = False
    assert bench.result_line(results, workloads.HEADLINE, 5)["verified"] is False
