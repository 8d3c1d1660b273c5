"""Builds the in-tree native libraries with hipcc / gcc (gfx950 only).

  nvshmem_amd/lib/libnvshmem_amd.so           host runtime + host-launched collectives (C ABI)
  nvshmem_amd/lib/libnvshmem_amd_perftest.so  kernels that call the device API + their C ABI drivers
  nvshmem_amd/lib/libnvshmem_amd_perftest_units.so  the in-kernel collective kernels of that library built with
                                              NVSHMEMI_AMD_UNIT_PACKETS (64-byte line packets), for their parity test
  oracle/liboracle.so                         CPU oracle (test infrastructure only)

Run as ``python -m nvshmem_amd.build``.  hipcc cross-compiles without a GPU.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "nvshmem_amd", "csrc")
LIBDIR = os.path.join(ROOT, "nvshmem_amd", "lib")
OBJDIR = os.path.join(ROOT, "build", "obj")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + INCLUDE, "-I" + CSRC,
]

RUNTIME_SOURCES = ["mspace.cpp", "runtime.hip", "teams.cpp", "collectives.hip", "host_rma.hip"]
PERFTEST_SOURCES = ["perftest/rma_kernels.hip", "perftest/coll_kernels.hip",
                    "perftest/moe_shuffle.hip", "perftest/moe_rowsignal.hip", "perftest/api_matrix.hip",
                    "perftest/amo_kernels.hip"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l)  # host pass does not know the GPU feature
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        sys.stderr.write(out + "\n")


UNITS_SOURCE = "perftest/coll_kernels.hip"     # built a second time with the line packets compiled in
UNITS_TAG = "+units"


def _compile(src):
    extra = []
    if src.endswith(UNITS_TAG):
        src, extra = src[:-len(UNITS_TAG)], ["-DNVSHMEMI_AMD_UNIT_PACKETS"]
    obj = os.path.join(OBJDIR, src.replace("/", "_") + ("_units" if extra else "") + ".o")
    cmd = [HIPCC] + HIP_FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    if src.endswith(".cpp"):
        cmd.insert(1, "-x")
        cmd.insert(2, "hip")
    _run(cmd)
    return obj


def _link(objs, out, extra=()):
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs + list(extra))


BINDIR = os.path.join(ROOT, "nvshmem_amd", "bin")
DRIVER_SOURCE = "perftest/perftest_main.cpp"   # command-line driver over both libraries
EXAMPLES = os.path.join(ROOT, "nvshmem_amd", "examples")   # user programs: public headers + the library only


def _build_example(name):
    """One command, as a user of the library would write it."""
    out = os.path.join(BINDIR, "examples", name)
    _run([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-I" + INCLUDE,
          os.path.join(EXAMPLES, name + ".hip"), "-o", out, "-L" + LIBDIR, "-lnvshmem_amd",
          "-Wl,-rpath,$ORIGIN/../../lib"])
    return out


def build_native(jobs=8):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    os.makedirs(BINDIR, exist_ok=True)
    sources = RUNTIME_SOURCES + [s for s in PERFTEST_SOURCES + [DRIVER_SOURCE]
                                 if os.path.exists(os.path.join(CSRC, s))]
    if UNITS_SOURCE in sources:
        sources.append(UNITS_SOURCE + UNITS_TAG)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = dict(zip(sources, pool.map(_compile, sources)))
    runtime = os.path.join(LIBDIR, "libnvshmem_amd.so")
    _link([objs[s] for s in RUNTIME_SOURCES], runtime)
    perf = [objs[s] for s in PERFTEST_SOURCES if s in objs]
    if perf:
        _link(perf, os.path.join(LIBDIR, "libnvshmem_amd_perftest.so"),
              ["-L" + LIBDIR, "-lnvshmem_amd", "-Wl,-rpath,$ORIGIN"])
    if UNITS_SOURCE + UNITS_TAG in objs:
        # the same entry point names as the library above: bound inside the library, loaded on its own
        _link([objs[UNITS_SOURCE + UNITS_TAG]], os.path.join(LIBDIR, "libnvshmem_amd_perftest_units.so"),
              ["-L" + LIBDIR, "-lnvshmem_amd", "-Wl,-rpath,$ORIGIN", "-Wl,-Bsymbolic"])
    if perf and DRIVER_SOURCE in objs:
        _run([HIPCC, "--offload-arch=gfx950", "-o", os.path.join(BINDIR, "nvshmem_perftest"),
              objs[DRIVER_SOURCE], "-L" + LIBDIR, "-lnvshmem_amd_perftest", "-lnvshmem_amd",
              "-Wl,-rpath,$ORIGIN/../lib"])
    if os.path.isdir(EXAMPLES):
        os.makedirs(os.path.join(BINDIR, "examples"), exist_ok=True)
        names = sorted(f[:-4] for f in os.listdir(EXAMPLES) if f.endswith(".hip"))
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(_build_example, names))
    return runtime


def build_oracle():
    """The oracle is a checker for tests and the bench's CPU baseline; nothing shipped links it."""
    odir = os.path.join(ROOT, "oracle")
    _run(["make", "-C", odir, "-B", "-s"])
    return os.path.join(odir, "liboracle.so")


def build_all():
    build_native()
    build_oracle()


if __name__ == "__main__":
    build_all()
    print("built:", ", ".join(sorted(os.listdir(LIBDIR))))
