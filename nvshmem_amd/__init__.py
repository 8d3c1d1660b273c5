"""MI355X-native NVSHMEM data-movement path: Python loader over the C ABI.

The product is the pair of shared libraries under ``nvshmem_amd/lib`` (built by
``python -m nvshmem_amd.build``); this package only loads them with ctypes and offers small
helpers for tests and the benchmark.  There is no CPU fallback: loading fails loudly when the
libraries are missing.
"""
from . import _lib, hip  # noqa: F401
from ._lib import load, load_perftest, LibraryMissing  # noqa: F401
from .host import (  # noqa: F401
    DTYPES, OPS, CMP, SIGNAL_SET, SIGNAL_ADD, TEAM_WORLD, SCOPE_THREAD, SCOPE_WARP, SCOPE_BLOCK,
    Runtime,
)
