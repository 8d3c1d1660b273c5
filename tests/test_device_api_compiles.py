"""Every family of device entry points that the reference's device headers stamp
(src/include/device/nvshmem_defines.h, nvshmemx_defines.h, nvshmem_coll_defines.cuh,
nvshmemx_coll_defines.cuh) exists under the same name in include/nvshmem.h: a translation unit that
takes the address of one representative of each family (one type, every scope) is compiled for
gfx950.  Compile only - no GPU is needed."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _names():
    names = []
    t = "int"
    for f in "put get put_nbi get_nbi p g iput iget put_signal put_signal_nbi".split():
        names.append("nvshmem_%s_%s" % (t, f))
    for f in "put get put_nbi get_nbi iput iget put_signal put_signal_nbi".split():
        for sc in ("warp", "block"):
            names.append("nvshmemx_%s_%s_%s" % (t, f, sc))
    for b in (8, 16, 32, 64, 128):
        for f in ("put%d", "get%d", "put%d_nbi", "get%d_nbi", "iput%d", "iget%d", "put%d_signal", "put%d_signal_nbi"):
            names.append("nvshmem_" + f % b)
            for sc in ("warp", "block"):
                names.append("nvshmemx_" + f % b + "_" + sc)
    for f in ("putmem", "getmem", "putmem_nbi", "getmem_nbi", "putmem_signal", "putmem_signal_nbi"):
        names.append("nvshmem_" + f)
        names += ["nvshmemx_%s_%s" % (f, sc) for sc in ("warp", "block")]
    for sc in ("warp", "block"):
        names += ["nvshmemx_%s_%s" % (f, sc) for f in (
            "barrier_all", "barrier", "sync_all", "team_sync", "alltoallmem", "broadcastmem", "fcollectmem",
            "int_alltoall", "int_broadcast", "int_fcollect", "int_sum_reduce", "uint_xor_reduce",
            "float_max_reduce", "half_prod_reduce", "bfloat16_min_reduce", "int_sum_reducescatter",
            "double_max_reducescatter")]
    names += ["nvshmemx_signal_op", "nvshmem_signal_fetch", "nvshmem_signal_wait_until",
              "nvshmem_info_get_name", "nvshmem_info_get_version", "nvshmemx_vendor_get_version_info",
              "nvshmem_barrier", "nvshmem_barrier_all", "nvshmem_sync_all", "nvshmem_team_sync",
              "nvshmem_alltoallmem", "nvshmem_broadcastmem", "nvshmem_fcollectmem", "nvshmem_int_alltoall",
              "nvshmem_int_broadcast", "nvshmem_int_fcollect", "nvshmem_int_sum_reduce",
              "nvshmem_int_sum_reducescatter", "nvshmem_quiet", "nvshmem_fence", "nvshmem_ptr", "nvshmem_my_pe",
              "nvshmem_n_pes", "nvshmem_team_my_pe", "nvshmem_team_n_pes", "nvshmem_team_translate_pe",
              "nvshmemx_double2_maxloc_reduce_block", "nvshmemx_barrier_warpgroup"]
    for f in ("wait_until", "wait_until_all", "wait_until_any", "wait_until_some", "wait_until_all_vector",
              "wait_until_any_vector", "wait_until_some_vector", "test", "test_all", "test_any", "test_some",
              "test_all_vector", "test_any_vector", "test_some_vector"):
        names.append("nvshmem_uint64_" + f)
    amo = lambda ty, op: "nvshmem_" + ty + "_atomic_" + op
    for op in ("fetch", "set", "swap"):
        names += [amo("long", op), amo("double", op)]
    for op in ("compare_swap", "fetch_add", "add", "fetch_inc", "inc"):
        names.append(amo("ptrdiff", op))
    for op in ("fetch_and", "and", "fetch_or", "or", "fetch_xor", "xor"):
        names.append(amo("uint32", op))
    return sorted(set(names))


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc is not installed")
def test_every_device_entry_point_family_compiles(tmp_path):
    names = _names()
    assert len(names) > 250
    src = '#include <hip/hip_runtime.h>\n#include "nvshmem.h"\n#include "nvshmemx.h"\n'
    src += "__global__ void probe(void **out) {\n"
    for i, n in enumerate(names):
        src += "    out[%d] = (void *)&%s;\n" % (i, n)
    src += "}\n"
    path = tmp_path / "probe.hip"
    path.write_text(src)
    proc = subprocess.run([HIPCC, "--offload-arch=gfx950", "-std=c++17", "--cuda-device-only",
                           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-ferror-limit=0",
                           "-I", os.path.join(ROOT, "include"), "-c", str(path), "-o", str(tmp_path / "probe.o")],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
    errors = [l for l in proc.stderr.decode().splitlines() if "error:" in l]
    assert proc.returncode == 0 and not errors, "\n".join(errors[:20])
