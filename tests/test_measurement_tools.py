"""The measurement tooling's arithmetic and parsing, checked on hand-made inputs (no GPU): the Little's-law
table of requests in flight, the driver-table parser of the put/get sweep, the kernel-source fingerprint
that ties a profile summary to the tree, and the rule that a summary of other sources yields no traffic."""
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from nvshmem_amd import fingerprint, perftest_tables, profile_summary  # noqa: E402


def test_requests_in_flight_by_littles_law():
    # 128 blocks of 1024 threads: 128 CUs busy for 1000 cycles per XCD (the counter sums the 8 XCDs);
    # 64000 reads that waited 1500 cycles each -> 64000 * 1500 / 1000 / 128 = 750 in flight per CU
    cs = {"GRBM_GUI_ACTIVE": 8000.0, "TCP_TCC_READ_REQ_sum": 64000.0, "TCP_TCC_READ_REQ_LATENCY_sum": 64000.0 * 1500,
          "TCP_TCC_WRITE_REQ_sum": 32000.0, "TCP_TCC_WRITE_REQ_LATENCY_sum": 32000.0 * 300}
    got = profile_summary.in_flight(cs, (16 * 1024, 1, 8, 1024))
    assert got["groups"] == 128 and got["cus"] == 128 and got["cycles"] == 1000.0
    assert got["reads"] == 750.0 and got["writes"] == 75.0
    assert got["read_latency"] == 1500.0 and got["write_latency"] == 300.0
    # a grid of more groups than the GPU has compute units is spread over all 256
    assert profile_summary.in_flight(cs, (64 * 4096, 1, 8, 64))["cus"] == 256
    # a pass without the latency counters gives no row
    assert profile_summary.in_flight({"GRBM_GUI_ACTIVE": 8000.0}, (64, 1, 1, 64)) is None


def test_driver_table_rows():
    text = "#shmem_put_bw\nsize(B)     scope     BW (GB/s per PE)\n8           block     0.002\n" \
           "268435456   block     382.40\nnot a row\n"
    assert perftest_tables.rows_of(text) == [(8, 0.002), (268435456, 382.40)]


def test_collective_table_rows_are_the_bandwidth_table_only():
    text = ("#reduction_on_stream\nsize(B)     scope     latency (us)\n1024        stream    3.24\n"
            "#reduction_on_stream\nsize(B)     scope     algorithmic BW (GB/s)\n1024        stream    5.05\n"
            "2048        stream    11.2\n")
    assert perftest_tables.bandwidth_rows(text) == [(1024, 5.05), (2048, 11.2)]


def test_fingerprint_covers_the_kernel_sources_and_is_stable():
    files = fingerprint.kernel_sources()
    assert "include/nvshmem_amd/device/nvshmemi_device.h" in files
    assert "nvshmem_amd/csrc/collectives.hip" in files
    assert "nvshmem_amd/csrc/perftest/moe_rowsignal.hip" in files
    fp = fingerprint.kernel_source_fingerprint()
    assert re.fullmatch(r"[0-9a-f]{16}", fp) and fp == fingerprint.kernel_source_fingerprint()


def test_traffic_is_quoted_only_from_a_summary_of_these_sources(tmp_path, monkeypatch):
    import bench
    summary = ("kernel_sources_fingerprint: %s\n"
               "measured_traffic_bytes: 100 read + 200 written = 0.0 MiB per launch of the dominant kernel\n")
    monkeypatch.setattr(bench, "ROOT", str(tmp_path), raising=False)
    prof = tmp_path / "profiles"
    prof.mkdir()
    (prof / "some_kernel__some_workload.txt").write_text(summary % "0123456789abcdef")
    assert bench.measured_traffic("some_workload", "0123456789abcdef") == 300
    assert bench.measured_traffic("some_workload", "fedcba9876543210") is None
    assert bench.measured_traffic("another_workload", "0123456789abcdef") is None
