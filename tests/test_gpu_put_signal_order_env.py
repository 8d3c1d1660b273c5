"""The library-wide order of put-with-signal as the environment sets it at nvshmem_init (a module of its
own: it initialises the library several times, which no other runtime may be alive for)."""
import os

import pytest

import nvshmem_amd as N
from gpu_util import note

pytestmark = pytest.mark.gpu


def test_put_signal_order_from_the_environment():
    for value, want in (("payload", 1), ("full", 0), ("nonsense", 0)):
        note("NVSHMEM_AMD_PUT_SIGNAL_ORDER=%s" % value)
        os.environ["NVSHMEM_AMD_PUT_SIGNAL_ORDER"] = value
        try:
            r = N.Runtime(npes=2, symmetric_size=8 << 20)
            try:
                assert r.lib.nvshmemx_amd_get_put_signal_order() == want, value
            finally:
                r.finalize()
        finally:
            del os.environ["NVSHMEM_AMD_PUT_SIGNAL_ORDER"]
    r = N.Runtime(npes=2, symmetric_size=8 << 20)
    try:
        assert r.lib.nvshmemx_amd_get_put_signal_order() == 0      # the default is the reference's order
    finally:
        r.finalize()
