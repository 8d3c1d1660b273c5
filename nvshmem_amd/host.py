"""Host-side helper over the C ABI: bring-up, symmetric buffers, per-PE transfers, collectives.

Names and argument meaning follow the C API (``nvshmem_<type>_<op>_reduce`` etc.); errors from the
library surface as exceptions carrying ``nvshmemx_amd_last_error()``.
"""
import ctypes as C

import numpy as np

from . import _lib, hip

TEAM_WORLD = 0
SIGNAL_SET, SIGNAL_ADD = 9, 10
CMP = {"EQ": 0, "NE": 1, "GT": 2, "LE": 3, "LT": 4, "GE": 5}
SCOPE_THREAD, SCOPE_WARP, SCOPE_BLOCK = 0, 1, 2

# element kinds / operators: numbering of nvshmemi_amd_dtype_t / nvshmemi_amd_op_t
DTYPES = {"i8": 0, "i16": 1, "i32": 2, "i64": 3, "u8": 4, "u16": 5, "u32": 6, "u64": 7,
          "f16": 8, "bf16": 9, "f32": 10, "f64": 11}
OPS = {"and": 0, "or": 1, "xor": 2, "min": 3, "max": 4, "sum": 5, "prod": 6}

# API type names -> (numpy storage dtype, element kind)
RMA_TYPES = {
    "bfloat16": (np.uint16, "bf16"), "half": (np.uint16, "f16"), "float": (np.float32, "f32"),
    "double": (np.float64, "f64"), "char": (np.int8, "i8"), "short": (np.int16, "i16"),
    "schar": (np.int8, "i8"), "int": (np.int32, "i32"), "long": (np.int64, "i64"),
    "longlong": (np.int64, "i64"), "uchar": (np.uint8, "u8"), "ushort": (np.uint16, "u16"),
    "uint": (np.uint32, "u32"), "ulong": (np.uint64, "u64"), "ulonglong": (np.uint64, "u64"),
    "int8": (np.int8, "i8"), "int16": (np.int16, "i16"), "int32": (np.int32, "i32"),
    "int64": (np.int64, "i64"), "uint8": (np.uint8, "u8"), "uint16": (np.uint16, "u16"),
    "uint32": (np.uint32, "u32"), "uint64": (np.uint64, "u64"), "size": (np.uint64, "u64"),
    "ptrdiff": (np.int64, "i64"),
}
WAIT_TYPES = ["short", "int", "long", "longlong", "ushort", "uint", "ulong", "ulonglong", "int32",
              "int64", "uint32", "uint64", "size", "ptrdiff"]
REDUCE_TYPES_BITWISE = ["uchar", "ushort", "uint", "ulong", "ulonglong", "int8", "int16", "int32",
                        "int64", "uint8", "uint16", "uint32", "uint64", "size"]
REDUCE_TYPES_STANDARD = REDUCE_TYPES_BITWISE + ["char", "schar", "short", "int", "long", "longlong",
                                                "bfloat16", "half", "float", "double"]


class NvshmemError(RuntimeError):
    pass


class Runtime:
    """One initialised logical-PE runtime.  Use as a context manager."""

    def __init__(self, npes=8, symmetric_size=1 << 30):
        self.lib = _lib.load()
        self.perf = None
        rc = self.lib.nvshmemx_amd_init(npes, symmetric_size)
        if rc != 0:
            raise NvshmemError("nvshmemx_amd_init(%d, %d) -> %d: %s"
                               % (npes, symmetric_size, rc, self.last_error()))
        self.npes = npes
        self.live = True

    # -- lifecycle ---------------------------------------------------------------------------
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.finalize()

    def finalize(self):
        if self.live:
            self.lib.nvshmem_finalize()
            self.live = False

    def last_error(self):
        return self.lib.nvshmemx_amd_last_error().decode()

    def perftest(self):
        if self.perf is None:
            self.perf = _lib.load_perftest()
        return self.perf

    # -- heap --------------------------------------------------------------------------------
    def malloc(self, nbytes):
        p = self.lib.nvshmem_malloc(nbytes)
        if not p and nbytes:
            raise NvshmemError("nvshmem_malloc(%d): %s" % (nbytes, self.last_error()))
        return p

    def calloc(self, count, size):
        p = self.lib.nvshmem_calloc(count, size)
        if not p and count * size:
            raise NvshmemError("nvshmem_calloc: %s" % self.last_error())
        return p

    def free(self, ptr):
        self.lib.nvshmem_free(ptr)

    def ptr(self, sym, pe):
        return self.lib.nvshmem_ptr(sym, pe)

    # -- teams ------------------------------------------------------------------------------
    def team_split_strided(self, parent, start, stride, size):
        t = C.c_int32(-1)
        rc = self.lib.nvshmem_team_split_strided(parent, start, stride, size, None, 0, C.byref(t))
        self._check(rc, "nvshmem_team_split_strided")
        return t.value

    def team_split_2d(self, parent, xrange_):
        x, y = C.c_int32(-1), C.c_int32(-1)
        rc = self.lib.nvshmem_team_split_2d(parent, xrange_, None, 0, C.byref(x), None, 0, C.byref(y))
        self._check(rc, "nvshmem_team_split_2d")
        return x.value, y.value

    def team_destroy(self, team):
        self.lib.nvshmem_team_destroy(team)

    def team_view(self, team, pe):
        """(start, stride, size, my_pe) of the team as world PE `pe` sees it; size 0: not a member."""
        v = (C.c_int32 * 4)()
        self._check(self.lib.nvshmemx_amd_team_view(team, pe, v), "nvshmemx_amd_team_view")
        return tuple(v)

    # -- plumbing: per-PE host <-> device transfers -----------------------------------------
    def upload(self, sym, pe, array, byte_offset=0):
        array = np.ascontiguousarray(array)
        hip.upload(self.ptr(sym, pe) + byte_offset, array)

    def upload_all(self, sym, arrays, byte_offset=0):
        """arrays[pe] (or a [npes, ...] array) -> every PE's copy."""
        for pe in range(self.npes):
            self.upload(sym, pe, arrays[pe], byte_offset)

    def download(self, sym, pe, shape, dtype, byte_offset=0):
        out = np.empty(shape, dtype=dtype)
        hip.download(out, self.ptr(sym, pe) + byte_offset)
        return out

    def download_all(self, sym, shape, dtype, byte_offset=0):
        return np.stack([self.download(sym, pe, shape, dtype, byte_offset) for pe in range(self.npes)])

    def fill(self, sym, value, nbytes):
        for pe in range(self.npes):
            hip.memset(self.ptr(sym, pe), value, nbytes)

    def sync(self):
        self.lib.nvshmem_barrier_all()

    # -- collectives (one call serves all PEs) ------------------------------------------------
    def _check(self, rc, what):
        if rc != 0:
            raise NvshmemError("%s -> %d: %s" % (what, rc, self.last_error()))

    def reduce(self, type_name, op, dest, src, nreduce, stream=None, team=TEAM_WORLD):
        if stream is None:
            name = "nvshmem_%s_%s_reduce" % (type_name, op)
            rc = _lib.typed_coll(self.lib, name)(team, dest, src, nreduce)
        else:
            name = "nvshmemx_%s_%s_reduce_on_stream" % (type_name, op)
            rc = _lib.typed_coll(self.lib, name, True)(team, dest, src, nreduce, stream.ptr)
        self._check(rc, name)

    def reducescatter(self, type_name, op, dest, src, nreduce, stream=None, team=TEAM_WORLD):
        if stream is None:
            name = "nvshmem_%s_%s_reducescatter" % (type_name, op)
            rc = _lib.typed_coll(self.lib, name)(team, dest, src, nreduce)
        else:
            name = "nvshmemx_%s_%s_reducescatter_on_stream" % (type_name, op)
            rc = _lib.typed_coll(self.lib, name, True)(team, dest, src, nreduce, stream.ptr)
        self._check(rc, name)

    def broadcast(self, type_name, dest, src, nelems, root, stream=None, team=TEAM_WORLD):
        if stream is None:
            name = "nvshmem_%s_broadcast" % type_name
            rc = _lib.typed_coll(self.lib, name, rooted=True)(team, dest, src, nelems, root)
        else:
            name = "nvshmemx_%s_broadcast_on_stream" % type_name
            rc = _lib.typed_coll(self.lib, name, True, True)(team, dest, src, nelems, root, stream.ptr)
        self._check(rc, name)

    def broadcastmem(self, dest, src, nbytes, root, stream=None, team=TEAM_WORLD):
        if stream is None:
            self._check(self.lib.nvshmem_broadcastmem(team, dest, src, nbytes, root), "broadcastmem")
        else:
            self._check(self.lib.nvshmemx_broadcastmem_on_stream(team, dest, src, nbytes, root,
                                                                 stream.ptr), "broadcastmem_on_stream")

    def fcollect(self, type_name, dest, src, nelems, stream=None, team=TEAM_WORLD):
        if stream is None:
            name = "nvshmem_%s_fcollect" % type_name
            rc = _lib.typed_coll(self.lib, name)(team, dest, src, nelems)
        else:
            name = "nvshmemx_%s_fcollect_on_stream" % type_name
            rc = _lib.typed_coll(self.lib, name, True)(team, dest, src, nelems, stream.ptr)
        self._check(rc, name)

    def alltoall(self, type_name, dest, src, nelems, stream=None, team=TEAM_WORLD):
        if stream is None:
            name = "nvshmem_%s_alltoall" % type_name
            rc = _lib.typed_coll(self.lib, name)(team, dest, src, nelems)
        else:
            name = "nvshmemx_%s_alltoall_on_stream" % type_name
            rc = _lib.typed_coll(self.lib, name, True)(team, dest, src, nelems, stream.ptr)
        self._check(rc, name)

    def fcollectmem(self, dest, src, nbytes, stream=None, team=TEAM_WORLD):
        if stream is None:
            self._check(self.lib.nvshmem_fcollectmem(team, dest, src, nbytes), "fcollectmem")
        else:
            self._check(self.lib.nvshmemx_fcollectmem_on_stream(team, dest, src, nbytes,
                                                                stream.ptr), "fcollectmem_on_stream")

    def alltoallmem(self, dest, src, nbytes, stream=None, team=TEAM_WORLD):
        if stream is None:
            self._check(self.lib.nvshmem_alltoallmem(team, dest, src, nbytes), "alltoallmem")
        else:
            self._check(self.lib.nvshmemx_alltoallmem_on_stream(team, dest, src, nbytes,
                                                                stream.ptr), "alltoallmem_on_stream")

    def read_timeout(self, pe):
        rec = (C.c_uint64 * 4)()
        flag = self.lib.nvshmemx_amd_read_timeout(pe, rec)
        return flag, list(rec)
