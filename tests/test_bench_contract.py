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
