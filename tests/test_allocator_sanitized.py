"""The product allocator (nvshmem_amd/csrc/mspace.cpp) under AddressSanitizer and UndefinedBehaviorSanitizer,
run in lock-step with the oracle's independent model of the reference's mspace
(src/host/mem/custom_malloc.cpp:74-237): tests/native/allocator_fuzz.cpp compares every returned address, the
free byte count and the free chunk count over random malloc / align / realloc / free sequences.  Host code
only; the sanitizer runtime is linked statically."""
import os
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SAN = ["-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"]


@pytest.fixture(scope="module")
def fuzzer():
    with tempfile.TemporaryDirectory() as tmp:
        objs = []
        for compiler, flags, src in (
                ("g++", ["-std=c++17"], os.path.join(ROOT, "tests", "native", "allocator_fuzz.cpp")),
                ("g++", ["-std=c++17"], os.path.join(ROOT, "nvshmem_amd", "csrc", "mspace.cpp")),
                ("gcc", ["-fopenmp"], os.path.join(ROOT, "oracle", "nvshmem_oracle.c"))):
            obj = os.path.join(tmp, os.path.basename(src) + ".o")
            subprocess.run([compiler] + flags + SAN + ["-I" + os.path.join(ROOT, "nvshmem_amd", "csrc"),
                                                       "-I" + os.path.join(ROOT, "oracle"), "-c", src, "-o", obj],
                           check=True)
            objs.append(obj)
        exe = os.path.join(tmp, "allocator_fuzz")
        subprocess.run(["g++", "-fsanitize=address,undefined", "-static-libasan", "-fopenmp"] + objs +
                       ["-lm", "-o", exe], check=True)
        yield exe


@pytest.mark.parametrize("seed", [1, 2, 3, 0xC0FFEE])
def test_allocator_matches_the_model_under_sanitizers(fuzzer, seed):
    out = subprocess.run([fuzzer, str(seed), "20000"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=300)
    assert out.returncode == 0, out.stderr.decode()[-2000:]
    assert out.stdout.decode().split()[:2] == ["ok", "20000"]
