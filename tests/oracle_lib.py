"""ctypes wrapper of oracle/liboracle.so - the CPU checker.  Imported by tests, the smoke run and
the benchmark's cpu_baseline leg only."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_PATH = os.path.join(ROOT, "oracle", "liboracle.so")

DT = {"i8": 0, "i16": 1, "i32": 2, "i64": 3, "u8": 4, "u16": 5, "u32": 6, "u64": 7,
      "f16": 8, "bf16": 9, "f32": 10, "f64": 11}
OP = {"and": 0, "or": 1, "xor": 2, "min": 3, "max": 4, "sum": 5, "prod": 6}
NP_STORAGE = {"i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64, "u8": np.uint8,
              "u16": np.uint16, "u32": np.uint32, "u64": np.uint64, "f16": np.uint16,
              "bf16": np.uint16, "f32": np.float32, "f64": np.float64}

_lib = None
vp, sz, u64, i32 = C.c_void_p, C.c_size_t, C.c_uint64, C.c_int


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_PATH):
        raise RuntimeError("%s missing: run `make -C oracle`" % _PATH)
    L = C.CDLL(_PATH)
    sig = {
        "oracle_dtype_size": (sz, [i32]),
        "oracle_set_threads": (None, [i32]),
        "oracle_get_threads": (i32, []),
        "oracle_splitmix64": (u64, [u64]),
        "oracle_rand_u64": (u64, [u64, u64, u64]),
        "oracle_fill_bytes": (None, [vp, sz, u64, u64]),
        "oracle_fill_u64": (None, [vp, sz, u64, u64]),
        "oracle_fill_i32_pm2p20": (None, [vp, sz, u64, u64]),
        "oracle_fill_f32_normal": (None, [vp, sz, u64, u64]),
        "oracle_fill_bf16_normal": (None, [vp, sz, u64, u64]),
        "oracle_fill_f16_normal": (None, [vp, sz, u64, u64]),
        "oracle_bf16_to_f32": (C.c_float, [C.c_uint16]),
        "oracle_f32_to_bf16": (C.c_uint16, [C.c_float]),
        "oracle_f16_to_f32": (C.c_float, [C.c_uint16]),
        "oracle_f32_to_f16": (C.c_uint16, [C.c_float]),
        "oracle_copy": (None, [vp, vp, sz]),
        "oracle_ring_put": (None, [vp, vp, i32, sz]),
        "oracle_ring_get": (None, [vp, vp, i32, sz]),
        "oracle_signal_op": (u64, [u64, u64, i32]),
        "oracle_compare_u64": (i32, [u64, i32, u64]),
        "oracle_compare_i64": (i32, [C.c_int64, i32, C.c_int64]),
        "oracle_ptr": (u64, [u64, u64, i32, u64, i32]),
        "oracle_reduce": (i32, [i32, i32, i32, sz, vp, vp]),
        "oracle_reducescatter": (i32, [i32, i32, i32, sz, vp, vp]),
        "oracle_maxloc_reduce": (None, [i32, sz, vp, vp]),
        "oracle_broadcast": (None, [i32, sz, i32, vp, vp]),
        "oracle_amo": (C.c_uint64, [i32, i32, C.c_uint64, C.c_uint64, C.c_uint64, vp]),
        "oracle_team_split_strided": (i32, [vp, i32, i32, i32, i32, vp]),
        "oracle_team_translate_pe": (i32, [vp, i32, vp]),
        "oracle_team_split_2d": (None, [vp, i32, i32, vp, vp]),
        "oracle_fcollect": (None, [i32, sz, vp, vp]),
        "oracle_alltoall": (None, [i32, sz, vp, vp]),
        "oracle_space_create": (vp, [u64, u64]),
        "oracle_space_destroy": (None, [vp]),
        "oracle_space_alloc": (u64, [vp, u64]),
        "oracle_space_align": (u64, [vp, u64, u64]),
        "oracle_space_free": (i32, [vp, u64]),
        "oracle_space_realloc": (u64, [vp, u64, u64, vp]),
        "oracle_space_free_bytes": (u64, [vp]),
        "oracle_space_free_chunks": (u64, [vp]),
        "oracle_moe_routing": (None, [vp, i32, i32, i32, C.c_double, u64, u64]),
        "oracle_moe_plan": (None, [vp, i32, i32, i32, i32, vp, vp, vp, vp, vp]),
        "oracle_moe_dispatch_one": (None, [vp, i32, vp, i32, i32, i32, sz, vp, vp]),
        "oracle_moe_combine_one": (None, [vp, i32, vp, i32, i32, sz, vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def _p(a):
    return a.ctypes.data


# ---- inputs --------------------------------------------------------------------------------
def fill(kind, n, seed, pe):
    """kind: bytes | u64 | i32 | f32 | bf16 | f16 -> numpy array of n elements."""
    L = lib()
    if kind == "bytes":
        out = np.empty(n, np.uint8); L.oracle_fill_bytes(_p(out), n, seed, pe)
    elif kind == "u64":
        out = np.empty(n, np.uint64); L.oracle_fill_u64(_p(out), n, seed, pe)
    elif kind == "i32":
        out = np.empty(n, np.int32); L.oracle_fill_i32_pm2p20(_p(out), n, seed, pe)
    elif kind == "f32":
        out = np.empty(n, np.float32); L.oracle_fill_f32_normal(_p(out), n, seed, pe)
    elif kind == "bf16":
        out = np.empty(n, np.uint16); L.oracle_fill_bf16_normal(_p(out), n, seed, pe)
    elif kind == "f16":
        out = np.empty(n, np.uint16); L.oracle_fill_f16_normal(_p(out), n, seed, pe)
    else:
        raise ValueError(kind)
    return out


def fill_all(kind, npes, n, seed):
    return np.stack([fill(kind, n, seed, pe) for pe in range(npes)])


# ---- operators -----------------------------------------------------------------------------
def reduce(dtype, op, src):
    """src: [npes, n] array in the storage dtype of `dtype` -> [n] result of one PE."""
    src = np.ascontiguousarray(src)
    npes, n = src.shape
    out = np.empty(n, dtype=src.dtype)
    rc = lib().oracle_reduce(DT[dtype], OP[op], npes, n, _p(src), _p(out))
    if rc != 0:
        raise ValueError("oracle_reduce: %s/%s undefined" % (dtype, op))
    return out


def reducescatter(dtype, op, src):
    """src: [npes, npes*n] -> [npes, n]."""
    src = np.ascontiguousarray(src)
    npes, total = src.shape
    n = total // npes
    out = np.empty((npes, n), dtype=src.dtype)
    rc = lib().oracle_reducescatter(DT[dtype], OP[op], npes, n, _p(src), _p(out))
    if rc != 0:
        raise ValueError("oracle_reducescatter: %s/%s undefined" % (dtype, op))
    return out


def maxloc_reduce(src):
    """src: [npes, n, 2] float64 (value, location) -> [npes, n, 2]."""
    src = np.ascontiguousarray(src, dtype=np.float64)
    out = np.empty_like(src)
    lib().oracle_maxloc_reduce(src.shape[0], src.shape[1], _p(src), _p(out))
    return out


def broadcast(src_bytes, root):
    src = np.ascontiguousarray(src_bytes, dtype=np.uint8)
    out = np.empty_like(src)
    lib().oracle_broadcast(src.shape[0], src.shape[1], root, _p(src), _p(out))
    return out


AMO = {"inc": 2, "set": 3, "add": 4, "and": 5, "or": 6, "xor": 7, "fetch": 12, "fetch_inc": 13,
       "fetch_add": 14, "fetch_and": 15, "fetch_or": 16, "fetch_xor": 17, "swap": 18, "compare_swap": 19}


def amo(op, bits, current, value=0, cond=0):
    """-> (new contents, fetched value) of one atomic operation on a `bits`-bit word."""
    fetched = C.c_uint64(0)
    new = lib().oracle_amo(AMO[op], bits, current & (2**64 - 1), value & (2**64 - 1), cond & (2**64 - 1),
                           C.addressof(fetched))
    return int(new), int(fetched.value)


def _triple(t):
    return np.ascontiguousarray(t, dtype=np.int32)


def team_split_strided(parent, npes_world, start, stride, size):
    """(start, stride, size) of the child in world PEs, or None when the arguments are rejected."""
    child = np.empty(3, np.int32)
    par = _triple(parent)
    rc = lib().oracle_team_split_strided(_p(par), npes_world, start, stride, size, _p(child))
    return None if rc else tuple(int(v) for v in child)


def team_translate_pe(src, src_pe, dst):
    a, b = _triple(src), _triple(dst)
    return lib().oracle_team_translate_pe(_p(a), src_pe, _p(b))


def team_split_2d(parent, xrange_, index):
    x = np.empty(3, np.int32); y = np.empty(3, np.int32)
    par = _triple(parent)
    lib().oracle_team_split_2d(_p(par), xrange_, index, _p(x), _p(y))
    return tuple(int(v) for v in x), tuple(int(v) for v in y)


def team_members(team):
    start, stride, size = team
    return [start + i * stride for i in range(size)]


def fcollect(src_bytes):
    """src: [npes, seg] uint8 -> [npes, npes*seg]."""
    src = np.ascontiguousarray(src_bytes, dtype=np.uint8)
    npes, seg = src.shape
    out = np.empty((npes, npes * seg), np.uint8)
    lib().oracle_fcollect(npes, seg, _p(src), _p(out))
    return out


def alltoall(src_bytes):
    """src: [npes, npes*seg] uint8 -> [npes, npes*seg]."""
    src = np.ascontiguousarray(src_bytes, dtype=np.uint8)
    npes, total = src.shape
    out = np.empty_like(src)
    lib().oracle_alltoall(npes, total // npes, _p(src), _p(out))
    return out


def ring_put(src_bytes, out=None):
    src = np.ascontiguousarray(src_bytes, dtype=np.uint8)
    if out is None:
        out = np.empty_like(src)
    assert out.shape == src.shape and out.dtype == np.uint8 and out.flags.c_contiguous
    lib().oracle_ring_put(_p(out), _p(src), src.shape[0], src.shape[1])
    return out


def ring_get(src_bytes):
    src = np.ascontiguousarray(src_bytes, dtype=np.uint8)
    out = np.empty_like(src)
    lib().oracle_ring_get(_p(out), _p(src), src.shape[0], src.shape[1])
    return out


# ---- MoE -----------------------------------------------------------------------------------
def moe_routing(npes, tokens, topk, num_experts, zipf_s, seed):
    out = np.empty((npes, tokens * topk), np.int32)
    for pe in range(npes):
        row = np.empty(tokens * topk, np.int32)
        lib().oracle_moe_routing(_p(row), tokens, topk, num_experts, zipf_s, seed, pe)
        out[pe] = row
    return out


def moe_plan(experts, npes, tokens, topk, num_experts):
    experts = np.ascontiguousarray(experts, dtype=np.int32)
    counts = np.empty((npes, num_experts), np.int64)
    seg_base = np.empty((num_experts, npes), np.int64)
    dest_pe = np.empty((npes, tokens * topk), np.int32)
    dest_row = np.empty((npes, tokens * topk), np.int64)
    recv_rows = np.empty(npes, np.int64)
    lib().oracle_moe_plan(_p(experts), npes, tokens, topk, num_experts, _p(counts), _p(seg_base),
                          _p(dest_pe), _p(dest_row), _p(recv_rows))
    return counts, seg_base, dest_pe, dest_row, recv_rows


def moe_dispatch(send, dest_pe, dest_row, recv_rows, tokens, topk):
    """send: [npes, tokens, row_bytes] uint8 -> list of [recv_rows[pe], row_bytes] arrays."""
    send = np.ascontiguousarray(send, dtype=np.uint8)
    npes, _, row_bytes = send.shape
    out = []
    for pe in range(npes):
        buf = np.zeros((int(recv_rows[pe]), row_bytes), np.uint8)
        lib().oracle_moe_dispatch_one(_p(buf), pe, _p(send), npes, tokens, topk, row_bytes,
                                      _p(dest_pe), _p(dest_row))
        out.append(buf)
    return out


def moe_combine(recv_list, dest_pe, dest_row, tokens, topk, row_bytes):
    npes = len(recv_list)
    ptrs = (C.c_void_p * npes)(*[_p(r) for r in recv_list])
    out = np.empty((npes, tokens * topk, row_bytes), np.uint8)
    for src in range(npes):
        one = np.empty((tokens * topk, row_bytes), np.uint8)
        lib().oracle_moe_combine_one(_p(one), src, ptrs, tokens, topk, row_bytes, _p(dest_pe),
                                     _p(dest_row))
        out[src] = one
    return out
