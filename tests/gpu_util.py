"""Helpers shared by the GPU parity tests."""
import contextlib
import sys

import numpy as np

import nvshmem_amd as N


def note(*a):
    """Names the case before each GPU step, so a fault can be attributed from the log."""
    print("[case]", *a, file=sys.stderr, flush=True)


@contextlib.contextmanager
def runtime(npes, symmetric_size):
    note("nvshmemx_amd_init npes=%d symmetric_size=%d" % (npes, symmetric_size))
    rt = N.Runtime(npes=npes, symmetric_size=symmetric_size)
    try:
        yield rt
    finally:
        rt.finalize()


def bits_equal(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype.itemsize == b.dtype.itemsize and \
        np.array_equal(a.view(np.uint8), b.view(np.uint8))
