"""ctypes loading of the in-tree shared libraries and the C-ABI signatures used from Python."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.environ.get("NVSHMEM_AMD_LIBDIR") or os.path.join(ROOT, "nvshmem_amd", "lib")
INCLUDE = os.path.join(ROOT, "include")


class LibraryMissing(RuntimeError):
    pass


_cache = {}


def _open(name):
    if name in _cache:
        return _cache[name]
    path = os.path.join(LIBDIR, name)
    if not os.path.exists(path):
        raise LibraryMissing(
            "%s is not built; run `python -m nvshmem_amd.build` (there is no CPU fallback)" % path)
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    _cache[name] = lib
    return lib


vp, sz, u64, i32 = C.c_void_p, C.c_size_t, C.c_uint64, C.c_int


def load():
    """libnvshmem_amd.so with argument types set for the entry points Python calls."""
    lib = _open("libnvshmem_amd.so")
    if getattr(lib, "_typed", False):
        return lib
    sig = {
        "nvshmemx_amd_init": (i32, [i32, sz]),
        "nvshmem_init": (None, []),
        "nvshmem_finalize": (None, []),
        "nvshmemx_init_status": (i32, []),
        "nvshmem_my_pe": (i32, []),
        "nvshmem_n_pes": (i32, []),
        "nvshmem_init_thread": (i32, [i32, C.POINTER(i32)]),
        "nvshmem_query_thread": (None, [C.POINTER(i32)]),
        "nvshmemx_buffer_register": (i32, [vp, sz]),
        "nvshmemx_buffer_unregister": (i32, [vp]),
        "nvshmem_team_my_pe": (i32, [i32]),
        "nvshmem_team_n_pes": (i32, [i32]),
        "nvshmem_info_get_version": (None, [C.POINTER(i32), C.POINTER(i32)]),
        "nvshmem_info_get_name": (None, [C.c_char_p]),
        "nvshmem_malloc": (vp, [sz]),
        "nvshmem_calloc": (vp, [sz, sz]),
        "nvshmem_align": (vp, [sz, sz]),
        "nvshmem_free": (None, [vp]),
        "nvshmem_ptr": (vp, [vp, i32]),
        "nvshmem_quiet": (None, []),
        "nvshmem_fence": (None, []),
        "nvshmem_barrier_all": (None, []),
        "nvshmemx_amd_timeout_count": (u64, []),
        "nvshmem_barrier": (i32, [i32]),
        "nvshmem_sync_all": (None, []),
        "nvshmemx_barrier_all_on_stream": (None, [vp]),
        "nvshmem_putmem": (None, [vp, vp, sz, i32]),
        "nvshmem_getmem": (None, [vp, vp, sz, i32]),
        "nvshmemx_putmem_on_stream": (None, [vp, vp, sz, i32, vp]),
        "nvshmemx_getmem_on_stream": (None, [vp, vp, sz, i32, vp]),
        "nvshmemx_putmem_signal_on_stream": (None, [vp, vp, sz, vp, u64, i32, i32, vp]),
        "nvshmemx_signal_op_on_stream": (None, [vp, u64, i32, i32, vp]),
        "nvshmemx_signal_wait_until_on_stream": (None, [vp, i32, u64, vp]),
        "nvshmem_alltoallmem": (i32, [i32, vp, vp, sz]),
        "nvshmem_fcollectmem": (i32, [i32, vp, vp, sz]),
        "nvshmemx_alltoallmem_on_stream": (i32, [i32, vp, vp, sz, vp]),
        "nvshmemx_fcollectmem_on_stream": (i32, [i32, vp, vp, sz, vp]),
        "nvshmem_init_thread": (i32, [i32, C.POINTER(i32)]),
        "nvshmem_query_thread": (None, [C.POINTER(i32)]),
        "nvshmemx_buffer_register": (i32, [vp, sz]),
        "nvshmemx_buffer_unregister": (i32, [vp]),
        "nvshmem_team_my_pe": (i32, [i32]),
        "nvshmem_team_n_pes": (i32, [i32]),
        "nvshmem_team_translate_pe": (i32, [i32, i32, i32]),
        "nvshmem_team_split_strided": (i32, [i32, i32, i32, i32, vp, C.c_long, C.POINTER(i32)]),
        "nvshmem_team_split_2d": (i32, [i32, i32, vp, C.c_long, C.POINTER(i32), vp, C.c_long, C.POINTER(i32)]),
        "nvshmem_team_destroy": (None, [i32]),
        "nvshmem_team_get_config": (None, [i32, vp]),
        "nvshmemx_amd_team_view": (i32, [i32, i32, C.POINTER(i32)]),
        "nvshmem_team_sync": (i32, [i32]),
        "nvshmemx_team_sync_on_stream": (i32, [i32, vp]),
        "nvshmemx_barrier_on_stream": (i32, [i32, vp]),
        "nvshmem_broadcastmem": (i32, [i32, vp, vp, sz, i32]),
        "nvshmemx_broadcastmem_on_stream": (i32, [i32, vp, vp, sz, i32, vp]),
        "nvshmemx_amd_collective_launch": (i32, [vp] + [C.c_uint] * 6 + [vp, sz, vp]),
        "nvshmemx_amd_collective_launch_query_gridsize": (i32, [vp] + [C.c_uint] * 3 + [sz, C.POINTER(i32)]),
        "nvshmemx_amd_module_init": (i32, []),
        "nvshmemx_amd_set_spin_limit": (None, [u64]),
        "nvshmemx_amd_set_put_signal_order": (None, [i32]),
        "nvshmemx_amd_get_put_signal_order": (i32, []),
        "nvshmemx_amd_read_timeout": (u64, [i32, C.POINTER(u64)]),
        "nvshmemx_amd_last_error": (C.c_char_p, []),
        "nvshmemi_amd_mspace_create": (vp, [u64, u64]),
        "nvshmemi_amd_mspace_destroy": (None, [vp]),
        "nvshmemi_amd_mspace_allocate": (u64, [vp, u64]),
        "nvshmemi_amd_mspace_allocate_aligned": (u64, [vp, u64, u64]),
        "nvshmemi_amd_mspace_deallocate": (i32, [vp, u64]),
        "nvshmemi_amd_mspace_reallocate": (u64, [vp, u64, u64, C.POINTER(u64)]),
        "nvshmemi_amd_mspace_inuse_size": (u64, [vp, u64]),
        "nvshmemi_amd_mspace_free_bytes": (u64, [vp]),
        "nvshmemi_amd_mspace_free_chunks": (u64, [vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    lib._typed = True
    return lib


def typed_coll(lib, name, on_stream=False, rooted=False):
    """Typed collective entry point, e.g. nvshmem_float_sum_reduce / nvshmemx_int64_alltoall_on_stream;
    rooted adds the PE_root argument of broadcast."""
    fn = getattr(lib, name)
    fn.restype = i32
    fn.argtypes = [i32, vp, vp, sz] + ([i32] if rooted else []) + ([vp] if on_stream else [])
    return fn


def load_perftest():
    load()
    lib = _open("libnvshmem_amd_perftest.so")
    if getattr(lib, "_typed", False):
        return lib
    sig = {
        "nvshmem_perftest_ring_rma": [vp, vp, sz, i32, i32, i32, i32, i32, vp],
        "nvshmem_perftest_plain_copy": [vp, vp, sz, vp],
        "nvshmem_perftest_stream_probe": [vp, sz, i32, i32, i32, vp],
        "nvshmem_perftest_profile_marker": [vp],
        "nvshmem_perftest_p_g": [vp, vp, u64, vp],
        "nvshmem_perftest_pe_identity": [vp, i32, vp],
        "nvshmem_perftest_api_matrix": [vp, vp, vp, vp, vp, i32, vp],
        "nvshmem_perftest_signal_op": [vp, u64, i32, i32, i32, vp],
        "nvshmem_perftest_signal_wait": [vp, i32, u64, vp, vp],
        "nvshmem_perftest_put_signal_pingpong": [vp, vp, sz, i32, i32, vp],
        "nvshmem_perftest_ring_reduce": [vp, vp, sz, vp, sz, i32, i32, vp],
        "nvshmem_perftest_unit_packets_compiled": [],
        "nvshmem_perftest_device_reduce": [i32, i32, vp, vp, sz, i32, i32, vp],
        "nvshmem_perftest_device_fcollect": [vp, vp, sz, i32, i32, vp],
        "nvshmem_perftest_amo_matrix_cases": [],
        "nvshmem_perftest_amo_matrix": [vp, vp, vp, vp, vp, vp],
        "nvshmem_perftest_amo_contend": [vp, vp, vp, i32, i32, i32, vp],
        "nvshmem_perftest_coll_sequence": [vp, vp, vp, i32, i32, i32, i32, i32, i32, vp],
        "nvshmem_perftest_device_team_coll": [i32, i32, vp, vp, sz, i32, i32, i32, vp],
        "nvshmem_perftest_device_team_coll_loop": [i32, i32, vp, vp, sz, i32, i32, i32, i32, vp],
        "nvshmem_perftest_team_query": [vp, i32, i32, vp],
        "nvshmem_perftest_device_warpgroup_barrier": [vp, vp, i32, i32, i32, i32, vp],
        "nvshmem_perftest_device_team_barrier": [vp, vp, i32, i32, i32, i32, vp],
        "nvshmem_perftest_device_reducescatter": [i32, i32, vp, vp, sz, i32, i32, vp],
        "nvshmem_perftest_device_broadcast": [vp, vp, sz, i32, i32, i32, vp],
        "nvshmem_perftest_device_alltoall": [vp, vp, sz, i32, i32, vp],
        "nvshmem_perftest_device_barrier": [vp, vp, i32, i32, i32, vp],
        "nvshmem_perftest_device_maxloc": [i32, vp, vp, sz, i32, i32, vp, vp],
        "nvshmem_perftest_fill_words": [vp, u64, sz, vp],
        "nvshmem_perftest_pt2pt_latency": [i32, vp, vp, sz, i32, i32, vp],
        "nvshmem_perftest_element_bw": [i32, i32, vp, vp, sz, i32, i32, vp],
        "nvshmem_perftest_moe_dispatch": [vp, sz, vp, vp, vp, vp, vp, i32, i32, sz, i32, i32, vp],
        "nvshmem_perftest_moe_dispatch_ex": [vp, sz, vp, vp, vp, vp, vp, i32, i32, sz, i32, i32, i32, vp],
        "nvshmem_perftest_put_signal_stream": [vp, vp, vp, vp, sz, i32, i32, i32, i32, i32, vp],
        "nvshmem_perftest_moe_dispatch_put_signal": [vp, sz, vp, vp, vp, vp, vp, i32, i32, i32, sz, i32, i32, i32, vp],
        "nvshmem_perftest_moe_dispatch_pieces": [vp, sz, vp, vp, vp, vp, vp, i32, i32, sz, i32, i32, vp],
        "nvshmem_perftest_static_init": [],
        "nvshmem_perftest_moe_dispatch_pieces_static": [vp, sz, vp, vp, vp, vp, i32, i32, sz, i32, i32, vp],
        "nvshmem_perftest_moe_combine": [vp, vp, sz, vp, vp, i32, i32, sz, i32, i32, vp],
        "nvshmem_perftest_moe_combine_ex": [vp, vp, sz, vp, vp, i32, i32, sz, i32, i32, i32, vp],
        "nvshmem_perftest_moe_combine_pieces": [vp, vp, sz, vp, vp, i32, i32, sz, i32, i32, i32, i32, vp],
        "nvshmem_perftest_moe_exchange_offsets": [vp, vp, vp, i32, vp],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = i32, args
    lib._typed = True
    lib._signatures = sig
    return lib


def load_perftest_units():
    """The in-kernel collective test kernels built with NVSHMEMI_AMD_UNIT_PACKETS: same entry point names as
    in load_perftest(), so the library is opened on its own (RTLD_LOCAL) and only those names are typed."""
    main = load_perftest()
    name = "libnvshmem_amd_perftest_units.so"
    if name in _cache:
        return _cache[name]
    path = os.path.join(LIBDIR, name)
    if not os.path.exists(path):
        raise LibraryMissing(
            "%s is not built; run `python -m nvshmem_amd.build` (there is no CPU fallback)" % path)
    lib = C.CDLL(path, mode=C.RTLD_LOCAL)
    for fname, args in main._signatures.items():
        if hasattr(lib, fname):
            fn = getattr(lib, fname)
            fn.restype, fn.argtypes = i32, args
    _cache[name] = lib
    return lib


def declared_symbols(header_paths=None):
    """Names of every function the public headers declare as host entry points (macro-stamped ones
    expanded), for the export check."""
    from .host import RMA_TYPES, REDUCE_TYPES_BITWISE, REDUCE_TYPES_STANDARD, WAIT_TYPES
    names = set()
    text = open(os.path.join(INCLUDE, "nvshmem_amd", "nvshmem_host_api.h")).read()
    # drop the macro bodies, then collect plain declarations
    plain = re.sub(r"#define[^\n]*(\\\n[^\n]*)*", "", text)
    for m in re.finditer(r"NVSHMEMI_HOST_ONLY\s+[\w\s\*]+?\b(nvshmem\w+)\s*\(", plain):
        names.add(m.group(1))
    for t in RMA_TYPES:
        for form in ("put", "get", "put_nbi", "get_nbi", "p", "g", "iput", "iget"):
            names.add("nvshmem_%s_%s" % (t, form))
            names.add("nvshmemx_%s_%s_on_stream" % (t, form))
        names.update({"nvshmemx_%s_put_signal_on_stream" % t, "nvshmemx_%s_put_signal_nbi_on_stream" % t,
                      "nvshmem_%s_alltoall" % t, "nvshmem_%s_fcollect" % t,
                      "nvshmemx_%s_alltoall_on_stream" % t, "nvshmemx_%s_fcollect_on_stream" % t,
                      "nvshmem_%s_broadcast" % t, "nvshmemx_%s_broadcast_on_stream" % t})
    for bits in (8, 16, 32, 64, 128):
        for form in ("put%d", "get%d", "put%d_nbi", "get%d_nbi", "iput%d", "iget%d"):
            names.add("nvshmem_" + form % bits)
            names.add("nvshmemx_" + form % bits + "_on_stream")
        names.update({"nvshmemx_put%d_signal_on_stream" % bits, "nvshmemx_put%d_signal_nbi_on_stream" % bits})
    for t in WAIT_TYPES:
        names.update({"nvshmemx_%s_wait_until_on_stream" % t, "nvshmemx_%s_wait_until_all_on_stream" % t,
                      "nvshmemx_%s_wait_until_all_vector_on_stream" % t})
    bitwise = ["uint", "ulong", "ulonglong", "int32", "int64", "uint32", "uint64"]
    standard = bitwise + ["int", "long", "longlong", "size", "ptrdiff"]
    for t in standard + ["float", "double"]:
        names.update("nvshmem_%s_atomic_%s" % (t, op) for op in ("fetch", "set", "swap"))
    for t in standard:
        names.update("nvshmem_%s_atomic_%s" % (t, op)
                     for op in ("compare_swap", "fetch_add", "add", "fetch_inc", "inc"))
    for t in bitwise:
        names.update("nvshmem_%s_atomic_%s" % (t, op)
                     for op in ("fetch_and", "fetch_or", "fetch_xor", "and", "or", "xor"))
    for op in ("and", "or", "xor"):
        for t in REDUCE_TYPES_BITWISE:
            names.update({"nvshmem_%s_%s_reduce" % (t, op), "nvshmemx_%s_%s_reduce_on_stream" % (t, op),
                          "nvshmem_%s_%s_reducescatter" % (t, op),
                          "nvshmemx_%s_%s_reducescatter_on_stream" % (t, op)})
    for op in ("max", "min", "sum", "prod"):
        for t in REDUCE_TYPES_STANDARD:
            names.update({"nvshmem_%s_%s_reduce" % (t, op), "nvshmemx_%s_%s_reduce_on_stream" % (t, op),
                          "nvshmem_%s_%s_reducescatter" % (t, op),
                          "nvshmemx_%s_%s_reducescatter_on_stream" % (t, op)})
    perf = open(os.path.join(INCLUDE, "nvshmem_perftest.h")).read()
    perf_names = set(re.findall(r"\bint\s+(nvshmem_perftest_\w+)\s*\(", perf))
    return names, perf_names
