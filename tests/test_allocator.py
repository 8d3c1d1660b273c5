"""Symmetric-space allocator through the C ABI (no GPU): golden traces, differential test against
the oracle's independent model, and structural invariants.
Reference behaviour: class mspace, src/host/mem/custom_malloc.cpp:74-237."""
import ctypes as C
import json
import os

import numpy as np
import pytest

import oracle_lib as O
from nvshmem_amd import _lib

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "allocator_traces.json")


class Product:
    def __init__(self, base, cap):
        self.L = _lib.load()
        self.h = self.L.nvshmemi_amd_mspace_create(base, cap)

    def alloc(self, n):
        return self.L.nvshmemi_amd_mspace_allocate(self.h, n)

    def align(self, a, n):
        return self.L.nvshmemi_amd_mspace_allocate_aligned(self.h, a, n)

    def free(self, addr):
        return self.L.nvshmemi_amd_mspace_deallocate(self.h, addr)

    def free_bytes(self):
        return self.L.nvshmemi_amd_mspace_free_bytes(self.h)

    def free_chunks(self):
        return self.L.nvshmemi_amd_mspace_free_chunks(self.h)

    def size_of(self, addr):
        return self.L.nvshmemi_amd_mspace_inuse_size(self.h, addr)

    def realloc(self, addr, n):
        moved = C.c_uint64(0)
        r = self.L.nvshmemi_amd_mspace_reallocate(self.h, addr, n, C.byref(moved))
        return r, moved.value

    def close(self):
        self.L.nvshmemi_amd_mspace_destroy(self.h)


class Model:
    def __init__(self, base, cap):
        self.L = O.lib()
        self.h = self.L.oracle_space_create(base, cap)

    def alloc(self, n):
        return self.L.oracle_space_alloc(self.h, n)

    def align(self, a, n):
        return self.L.oracle_space_align(self.h, a, n)

    def free(self, addr):
        return self.L.oracle_space_free(self.h, addr)

    def realloc(self, addr, n):
        moved = C.c_uint64(0)
        r = self.L.oracle_space_realloc(self.h, addr, n, C.byref(moved))
        return r, moved.value

    def free_bytes(self):
        return self.L.oracle_space_free_bytes(self.h)

    def free_chunks(self):
        return self.L.oracle_space_free_chunks(self.h)

    def close(self):
        self.L.oracle_space_destroy(self.h)


def _replay(impl_cls, trace):
    base = trace["base"]
    impl = impl_cls(base, trace["capacity"])
    try:
        for i, st in enumerate(trace["steps"]):
            if st["op"] == "alloc":
                got = impl.alloc(st["bytes"])
                got = got - base if got else -1
            elif st["op"] == "align":
                got = impl.align(st["alignment"], st["bytes"])
                got = got - base if got else -1
            elif st["op"] == "realloc":
                got, moved = impl.realloc(base + st["addr"], st["bytes"])
                got = got - base if got else -1
                assert (moved - base if moved else -1) == st["moved"], "%s step %d %r moved %d" % (trace["name"], i, st, moved)
            else:
                got = impl.free(base + st["addr"])
            assert got == st["expect"], "%s step %d %r -> %d" % (trace["name"], i, st, got)
    finally:
        impl.close()


@pytest.mark.parametrize("impl", [Product, Model], ids=["library", "oracle-model"])
def test_golden_traces(impl):
    for trace in json.load(open(GOLDEN))["traces"]:
        _replay(impl, trace)


@pytest.mark.parametrize("seed", range(6))
def test_differential_random_traces(seed):
    rng = np.random.default_rng(seed)
    base, cap = 0x7F00_0000_0000 + int(rng.integers(0, 4)) * 128, 1 << 22
    a, b = Product(base, cap), Model(base, cap)
    live = []
    try:
        for step in range(3000):
            r = rng.random()
            if r < 0.5 or not live:
                n = int(rng.choice([1, 100, 512, 513, 4096, 70000, 300000]))
                if rng.random() < 0.25:
                    al = int(rng.choice([8, 64, 512, 4096, 65536]))
                    pa, pb = a.align(al, n), b.align(al, n)
                    if pa:
                        assert pa % al == 0
                else:
                    pa, pb = a.alloc(n), b.alloc(n)
                assert pa == pb, (step, n)
                if pa:
                    assert pa % 512 == 0 or pa % 8 == 0
                    live.append(pa)
            elif r < 0.65:
                k = int(rng.integers(0, len(live)))
                n = int(rng.choice([1, 300, 512, 2000, 4096, 50000, 200000]))
                (pa, ma), (pb, mb) = a.realloc(live[k], n), b.realloc(live[k], n)
                assert (pa, ma) == (pb, mb), (step, n)
                if pa:
                    live[k] = pa
            else:
                addr = live.pop(int(rng.integers(0, len(live))))
                assert a.free(addr) == 0 and b.free(addr) == 0
            assert a.free_bytes() == b.free_bytes()
            assert a.free_chunks() == b.free_chunks()
        for addr in live:
            assert a.free(addr) == 0 and b.free(addr) == 0
        # everything returned: one chunk covering the whole space again
        assert a.free_chunks() == 1 and b.free_chunks() == 1
        skipped = (512 - base % 512) % 512
        assert a.free_bytes() == cap - skipped == b.free_bytes()
    finally:
        a.close(); b.close()


def test_blocks_never_overlap_and_sizes_are_rounded():
    a = Product(1 << 40, 1 << 20)
    blocks = []
    rng = np.random.default_rng(1)
    for _ in range(200):
        n = int(rng.integers(1, 5000))
        p = a.alloc(n)
        if not p:
            break
        sz = a.size_of(p)
        assert sz == (n + 511) // 512 * 512 and p % 512 == 0
        blocks.append((p, sz))
    blocks.sort()
    for (p0, s0), (p1, _) in zip(blocks, blocks[1:]):
        assert p0 + s0 <= p1
    a.close()


def test_reallocate_grow_shrink_move():
    base = 1 << 40
    a = Product(base, 1 << 16)
    p = a.alloc(1000)            # [0, 1024)
    q = a.alloc(512)             # [1024, 1536)
    r, moved = a.realloc(p, 600)  # shrink in place to 1024 -> same rounded size
    assert (r, moved) == (p, 0) and a.size_of(p) == 1024
    r, moved = a.realloc(p, 100)  # shrink to 512, tail freed
    assert (r, moved) == (p, 0) and a.size_of(p) == 512
    assert a.alloc(512) == base + 512          # the freed tail is the lowest hole
    assert a.free(base + 512) == 0
    r, moved = a.realloc(p, 1024)  # grow in place into the hole behind it
    assert (r, moved) == (p, 0) and a.size_of(p) == 1024
    r, moved = a.realloc(p, 4096)  # blocked by q: moves
    assert r == base + 1536 and moved == p and a.size_of(r) == 4096
    assert a.alloc(1024) == p       # old block is free again
    assert a.free(q) == 0
    a.close()


def test_out_of_space_and_bad_alignment_return_null():
    a = Product(1 << 40, 4096)
    assert a.alloc(4097) == 0
    assert a.alloc(2**64 - 1) == 0
    assert a.align(4096, 2**64 - 100) == 0
    assert a.align(0, 8) == 0 and a.align(24, 8) == 0
    assert a.alloc(4096) == 1 << 40
    assert a.alloc(1) == 0
    a.close()
