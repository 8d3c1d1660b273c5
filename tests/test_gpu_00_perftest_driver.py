"""The command-line performance driver: runs in a child process against the built libraries and
prints tables in the reference's perftest layout; the numbers are only checked for sanity here.

The file name makes pytest collect it first: a cooperative launch in the child is refused
("operation cannot be performed in the present state") once the parent process has made a
cooperative launch of its own, and every later test file does."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "nvshmem_amd", "bin", "nvshmem_perftest")


def _run(*args, exe=DRIVER, env=None):
    assert os.path.exists(exe), "run `python -m nvshmem_amd.build` first"
    proc = subprocess.run([exe] + list(args), stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=100,
                          env=dict(os.environ, **(env or {})))
    err = proc.stderr.decode()
    if proc.returncode != 0 and "cannot be performed in the present state" in err:
        pytest.skip("cooperative launches are held by another process on this GPU")
    assert proc.returncode == 0, err
    return proc.stdout.decode()


def _rows(text, job):
    """[(size, scope, value)] of the first table of `job`."""
    lines = text.splitlines()
    start = next(i for i, l in enumerate(lines) if l.strip() == "#" + job or l.split() == ["#" + job])
    rows = []
    for l in lines[start + 2:]:
        if l.startswith("#") or not l.strip():
            break
        size, scope, value = l.split()
        rows.append((int(size), scope, float(value)))
    return rows


def test_put_bw_and_collective_tables():
    out = _run("put_bw", "--min", "1k", "--max", "16m", "--iters", "10")
    rows = _rows(out, "shmem_put_bw")
    assert [r[0] for r in rows] == [1024 << i for i in range(15)] and all(r[1] == "block" for r in rows)
    assert rows[-1][2] > 100.0            # GB/s per PE at 16 MiB
    out = _run("reduce", "--min", "4k", "--max", "4m", "--iters", "10", "--npes", "8")
    lat = _rows(out, "reduction_on_stream")
    assert len(lat) == 11 and all(v > 0 for _, _, v in lat)
    out = _run("broadcast", "--min", "64", "--max", "64k", "--iters", "5", "--npes", "4")
    assert len(_rows(out, "bcast_on_stream")) == 11
    # the same calls captured in a HIP graph and replayed
    for test, job in (("reduce", "reduction_on_stream"), ("fcollect", "fcollect_on_stream"), ("alltoall", "alltoall_on_stream")):
        rows = _rows(_run(test, "--min", "64", "--max", "1m", "--iters", "10", "--graph"), job)
        assert len(rows) == 15 and all(r[1] == "graph" and 0.0 < r[2] < 1e4 for r in rows), rows


def test_host_rma_tables():
    out = _run("host_put_bw", "--min", "1k", "--max", "1m", "--iters", "10", "--npes", "2")
    rows = _rows(out, "put_on_stream")
    assert [r[0] for r in rows] == [1024 << i for i in range(11)] and all(v > 0 for _, _, v in rows)
    assert len(_rows(_run("host_get_bw", "--min", "64", "--max", "4k", "--iters", "5"), "get_on_stream")) == 7


def test_device_latency_tables():
    out = _run("coll_latency", "--min", "8", "--max", "512", "--iters", "50", "--scope", "warp")
    for job in ("reduction_latency", "reducescatter_latency", "fcollect_latency", "alltoall_latency", "bcast_latency"):
        rows = _rows(out, job)
        assert [r[0] for r in rows] == [8, 16, 32, 64, 128, 256, 512] and all(r[1] == "warp" for r in rows)
        assert all(0.0 < v < 1000.0 for _, _, v in rows), (job, rows)
    assert 0.0 < _rows(out, "redmaxloc_latency")[0][2] < 1000.0
    out = _run("barrier_latency", "--iters", "100")
    assert "barrier_latency" in out
    out = _run("sync_latency", "--iters", "100", "--scope", "thread")
    assert 0.0 < float(out.split()[-1]) < 1000.0 and out.split()[0] == "#sync_latency"


def test_host_synchronisation_and_allocator_tables():
    for test, jobs in (("barrier_on_stream", ("#barrier_all_on_stream", "#barrier_on_stream")),
                       ("sync_on_stream", ("#sync_all_on_stream", "#sync_on_stream"))):
        lines = _run(test, "--iters", "50", "--npes", "4").splitlines()
        assert (lines[0], lines[3]) == jobs
        assert all(0.0 < float(lines[i].split()[-1]) < 10000.0 for i in (2, 5))
    out = _run("malloc", "--min", "512", "--max", "64m", "--npes", "2")
    for job in ("nvshmem_malloc", "nvshmem_free"):
        rows = _rows(out, job)
        assert [r[0] for r in rows] == [512 << i for i in range(18)] and all(0.0 <= v < 1e5 for _, _, v in rows)


def test_element_wise_bandwidth_tables():
    for test, job, elem in (("p_bw", "shmem_p_bw", "8"), ("g_bw", "shmem_g_bw", "4"), ("st_bw", "shmem_st_bw", "1"),
                            ("atomic_bw", "shmem_atomic_bw", "8")):
        rows = _rows(_run(test, "--min", "1k", "--max", "4m", "--iters", "5", "--elem", elem), job)
        assert [r[0] for r in rows] == [1024 << i for i in range(13)] and all(r[1] == elem + "-byte" for r in rows)
        assert all(v > 0 for _, _, v in rows), (job, rows)
    proc = subprocess.run([DRIVER, "atomic_bw", "--elem", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=100)
    assert proc.returncode == 2 and b"atomics" in proc.stderr


def test_bad_arguments_are_refused():
    proc = subprocess.run([DRIVER, "nonsense"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=100)
    assert proc.returncode == 2 and b"usage" in proc.stderr


def test_point_to_point_latency_tables():
    out = _run("pt2pt_latency", "--min", "8", "--max", "4k", "--iters", "50")
    for job in ("shmem_put_latency", "shmem_get_latency", "shmem_put_signal_ping_pong_latency"):
        rows = _rows(out, job)
        assert [r[0] for r in rows] == [8 << i for i in range(10)]
        assert all(0.0 < v < 1000.0 for _, _, v in rows), (job, rows)
    for name in ("shmem_p_latency", "shmem_g_latency", "shmem_atomic_latency", "shmem_signal_ping_pong_latency",
                 "shmem_p_ping_pong_latency", "shmem_atomic_ping_pong_latency"):
        line = next(l for l in out.splitlines() if l.startswith(name))
        assert 0.0 < float(line.split()[-1]) < 1000.0, line


@pytest.mark.parametrize("name,npes", [("put_block", 8), ("ring_bcast", 8), ("ring_bcast", 3), ("allreduce", 8),
                                       ("allreduce", 5), ("on_stream", 8), ("on_stream", 16), ("moe_shuffle", 8), ("moe_shuffle", 3),
                                       ("collective_launch", 8), ("collective_launch", 5), ("thread_group", 8),
                                       ("thread_group", 3), ("simple_shift", 8), ("simple_shift", 2)])
def test_example_programs_reach_their_known_answers(name, npes):
    """nvshmem_amd/examples/*.hip are user programs built with one hipcc command against include/ and
    libnvshmem_amd.so; each checks the closed-form answer of the reference example it models on every
    PE and prints PASSED."""
    exe = os.path.join(ROOT, "nvshmem_amd", "bin", "examples", name)
    out = _run(exe=exe, env={"NVSHMEM_AMD_NPES": str(npes), "NVSHMEM_SYMMETRIC_SIZE": str(128 << 20)})
    assert out.strip().endswith(name + ": PASSED"), out
