"""GPU parity of the atomic memory operations: every stamped (type, operation) pair once on an
uncontended word against the oracle (bit-exact, value returned and word left behind), then all
threads of all PEs contending for the same words, checked through invariants that only hold if
every operation was atomic."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import note, runtime

pytestmark = pytest.mark.gpu

# type lists in the order of NVSHMEMI_REPT_FOR_*_AMO_TYPES (include/nvshmem_amd/nvshmem_types.h)
BITWISE = [("uint", 32), ("ulong", 64), ("ulonglong", 64), ("int32", 32), ("int64", 64),
           ("uint32", 32), ("uint64", 64)]
STANDARD = BITWISE + [("int", 32), ("long", 64), ("longlong", 64), ("size", 64), ("ptrdiff", 64)]
EXTENDED = [("float", 32), ("double", 64)]


def _cases():
    """(name, bits, operation, which cond) in the kernel's case order."""
    out = []
    for name, bits in STANDARD + EXTENDED:
        out += [(name, bits, "fetch", None), (name, bits, "set", None), (name, bits, "swap", None)]
    for name, bits in STANDARD:
        out += [(name, bits, "compare_swap", "hit"), (name, bits, "compare_swap", "miss"),
                (name, bits, "fetch_add", None), (name, bits, "add", None),
                (name, bits, "fetch_inc", None), (name, bits, "inc", None)]
    for name, bits in BITWISE:
        out += [(name, bits, op, None) for op in ("fetch_and", "and", "fetch_or", "or", "fetch_xor", "xor")]
    return out


FETCHING = {"fetch", "swap", "compare_swap", "fetch_add", "fetch_inc", "fetch_and", "fetch_or", "fetch_xor"}


@pytest.mark.parametrize("npes", [8, 3])
def test_every_amo_entry_point_once(npes):
    cases = _cases()
    rng = np.random.default_rng(npes)
    with runtime(npes, 1 << 22) as rt:
        perf = rt.perftest()
        k = perf.nvshmem_perftest_amo_matrix_cases()
        assert k == len(cases) == 3 * 14 + 6 * 12 + 6 * 7
        words = k + 1
        slots = rt.calloc(words, 8); val = rt.calloc(words, 8); cond = rt.calloc(words, 8)
        out = rt.calloc(words, 8); ncases = rt.calloc(1, 4)
        init = rng.integers(0, 2**64, (npes, words), dtype=np.uint64)
        vals = rng.integers(0, 2**64, (npes, words), dtype=np.uint64)
        # edge words for the first PEs: all ones (wraps on add / inc), zero, sign bits
        init[0, :] = 2**64 - 1
        if npes > 2:
            init[2, :] = 0
            vals[2, :] = 0x8000000080000000
        conds = np.empty_like(init)
        for pe in range(npes):
            target = (pe + 1) % npes          # PE pe acts on its right neighbour's slots
            for j, (name, bits, op, which) in enumerate(cases):
                m = np.uint64(2**bits - 1)
                conds[pe, j] = (init[target, j] & m) if which == "hit" else ((init[target, j] ^ np.uint64(1)) & m)
        rt.upload_all(slots, init); rt.upload_all(val, vals); rt.upload_all(cond, conds)
        note("amo matrix npes=%d cases=%d" % (npes, k))
        assert perf.nvshmem_perftest_amo_matrix(slots, val, cond, out, ncases, None) == 0
        rt.sync()
        assert (rt.download_all(ncases, (1,), np.int32) == k).all()
        got_slots = rt.download_all(slots, (words,), np.uint64)
        got_out = rt.download_all(out, (words,), np.uint64)
        for pe in range(npes):
            target = (pe + 1) % npes
            for j, (name, bits, op, which) in enumerate(cases):
                new, fetched = O.amo(op, bits, int(init[target, j]), int(vals[pe, j]), int(conds[pe, j]))
                m = 2**bits - 1
                # the bytes of the word above the type's width are untouched
                want_word = (int(init[target, j]) & ~m) | new
                assert int(got_slots[target, j]) == want_word, (pe, j, name, op, which)
                if op in FETCHING:
                    assert int(got_out[pe, j]) == fetched, (pe, j, name, op, which)
                else:
                    assert int(got_out[pe, j]) == 0, (pe, j, name, op)
        for p in (slots, val, cond, out, ncases):
            rt.free(p)


@pytest.mark.parametrize("home,blocks,threads", [(0, 64, 256), (5, 7, 96)])
def test_contended_amos_are_atomic(home, blocks, threads):
    npes = 8
    total = npes * blocks * threads
    with runtime(npes, 1 << 24) as rt:
        perf = rt.perftest()
        words = rt.calloc(8, 8); seen = rt.calloc(total, 4); chain = rt.calloc(total, 8)
        start = np.zeros(8, np.uint64)
        start[4] = 2**64 - 1                      # the word that is cleared bit by bit
        rt.upload(words, home, start)
        note("amo contend home=%d %d threads" % (home, total))
        assert perf.nvshmem_perftest_amo_contend(words, seen, chain, home, blocks, threads, None) == 0
        rt.sync()
        w = rt.download(words, home, (8,), np.uint64)
        assert int(w[0]) == total                                   # every fetch_add counted
        assert (rt.download(seen, home, (total,), np.uint32) == 1).all()   # tickets: a permutation
        assert 1 <= int(w[1]) <= total and int(w[7]) == 1           # one compare_swap winner
        ids = np.arange(total, dtype=np.uint64)
        bits = np.bitwise_xor.reduce(np.uint64(1) << (ids % np.uint64(64)))
        assert int(w[2]) == int(bits)                               # xor of all the bits
        present = np.bitwise_or.reduce(np.uint64(1) << (ids % np.uint64(64)))
        assert int(w[3]) == int(present) and int(w[4]) == (2**64 - 1) & ~int(present)
        assert int(w[5]) == (total * (total - 1) // 2) % 2**32      # 32-bit wrapping sum, upper half untouched
        # swap chain: the returned values are 0 (first) and every id + 1 except the last one stored
        c = rt.download(chain, home, (total,), np.uint64)
        assert sorted(int(x) for x in c) == sorted(set(range(total + 1)) - {int(w[6])})
        # the other PEs' copies were never touched
        other = (home + 1) % npes
        assert (rt.download(words, other, (8,), np.uint64) == 0).all()
        for p in (words, seen, chain):
            rt.free(p)
