"""The C-ABI libraries load without a GPU and export every entry point the headers declare."""
import ctypes as C
import os
import subprocess

import pytest

from nvshmem_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_runtime_library_exports_every_declared_symbol():
    lib = _lib.load()
    names, _ = _lib.declared_symbols()
    assert len(names) > 500, "header parse lost the stamped declarations (%d)" % len(names)
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, missing[:20]


def test_perftest_library_exports_every_declared_symbol():
    lib = _lib.load_perftest()
    _, names = _lib.declared_symbols()
    assert len(names) >= 15
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, missing


def test_constants_have_the_reference_abi_values():
    # compile a C program against the public header and print the enum values
    src = r'''
    #include <stdio.h>
    #include "nvshmem.h"
    int main(void) {
        printf("%d %d %d %d %d %d %d %d %d %d %zu %d %d %d %d %d %d %d %zu\n", NVSHMEM_CMP_EQ,
               NVSHMEM_CMP_NE, NVSHMEM_CMP_GT,
               NVSHMEM_CMP_LE, NVSHMEM_CMP_LT, NVSHMEM_CMP_GE, NVSHMEM_SIGNAL_SET, NVSHMEM_SIGNAL_ADD,
               NVSHMEM_TEAM_WORLD, NVSHMEMX_ERROR_INTERNAL, sizeof(nvshmemi_device_state_t),
               NVSHMEM_TEAM_INVALID, NVSHMEM_TEAM_SHARED, NVSHMEMX_TEAM_NODE,
               NVSHMEMX_TEAM_SAME_MYPE_NODE, NVSHMEMI_TEAM_SAME_GPU, NVSHMEMI_TEAM_GPU_LEADERS,
               NVSHMEM_TEAMS_MIN, sizeof(nvshmem_team_config_t));
        return 0;
    }'''
    exe = "/tmp/nvshmem_amd_abi_probe"
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-x", "c", "-", "-I",
                    os.path.join(ROOT, "include"), "-o", exe], input=src.encode(), check=True)
    out = subprocess.run([exe], stdout=subprocess.PIPE, check=True).stdout.decode().split()
    assert out[:10] == ["0", "1", "2", "3", "4", "5", "9", "10", "0", "7"]
    assert int(out[10]) == 112
    # team ids: src/include/device_host/nvshmem_common.cuh:406-419; the config struct is 64 bytes
    # (src/include/device_host/nvshmem_types.h:301)
    assert out[11:] == ["-1", "1", "2", "3", "4", "5", "6", "64"]


def test_api_before_init_reports_instead_of_crashing():
    lib = _lib.load()
    assert lib.nvshmemx_init_status() == 0           # NVSHMEM_STATUS_NOT_INITIALIZED
    assert lib.nvshmem_malloc(1024) is None
    assert b"before nvshmem_init" in lib.nvshmemx_amd_last_error()
    assert lib.nvshmem_ptr(0x1000, 0) is None
    assert lib.nvshmem_n_pes() == 0
    major, minor = C.c_int(), C.c_int()
    lib.nvshmem_info_get_version(C.byref(major), C.byref(minor))
    assert (major.value, minor.value) == (1, 3)      # OpenSHMEM spec level of the reference
    name = C.create_string_buffer(256)
    lib.nvshmem_info_get_name(name)
    assert name.value.startswith(b"NVSHMEM v3.5.1")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "LIBDIR", str(tmp_path))
    monkeypatch.setattr(_lib, "_cache", {})
    with pytest.raises(_lib.LibraryMissing):
        _lib.load()
