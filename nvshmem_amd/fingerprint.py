"""Fingerprint of the sources the GPU kernels are compiled from.

A profile summary under profiles/ records the fingerprint of the tree it was measured on; the benchmark
quotes a summary's measured HBM traffic only while the fingerprint still matches, so a kernel change
without a new profile shows up as "traffic": null instead of a stale figure.
"""
import hashlib
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KERNEL_SOURCE_DIRS = ("nvshmem_amd/csrc", "nvshmem_amd/csrc/perftest", "include/nvshmem_amd/device")
KERNEL_SOURCE_SUFFIXES = (".hip", ".h", ".hpp", ".cpp")


def kernel_sources():
    out = []
    for d in KERNEL_SOURCE_DIRS:
        full = os.path.join(ROOT, d)
        for f in sorted(os.listdir(full)):
            if f.endswith(KERNEL_SOURCE_SUFFIXES):
                out.append(os.path.join(d, f))
    return out


def kernel_source_fingerprint():
    """sha256 over (relative path, contents) of every kernel-bearing source file, first 16 hex digits."""
    h = hashlib.sha256()
    for rel in kernel_sources():
        h.update(rel.encode())
        with open(os.path.join(ROOT, rel), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]
