"""GPU parity on seeded random cases: host-launched collectives on random strided teams with random
element types, operators, counts and byte offsets, each compared with the CPU oracle bit for bit
(integers, copies) or bit for bit with the fixed PE order (floating point).  The cases are drawn from
a fixed seed, so a failure names a reproducible case.  NVSHMEM_AMD_TEST_SEED_OFFSET shifts the seeds for a longer
run over other cases; the kernel-selection thresholds can be lowered from the environment as for any program
(NVSHMEM_AMD_LDS_REDUCE_BYTES=0 NVSHMEM_AMD_CACHEABLE_SOURCE_BYTES=0 NVSHMEM_AMD_CHUNKED_COPY_BYTES=0 sends these
small messages through the
kernels meant for large ones)."""
import os

import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import bits_equal, note, runtime
from nvshmem_amd.host import REDUCE_TYPES_BITWISE, REDUCE_TYPES_STANDARD, RMA_TYPES

pytestmark = pytest.mark.gpu

SEED_OFFSET = int(os.environ.get("NVSHMEM_AMD_TEST_SEED_OFFSET", "0"))
CAP = 1 << 20          # bytes of source / destination per PE
GUARD = 256


def _random_values(rng, kind, shape, narrow=False):
    """narrow: magnitudes in [0.5, 2), so that a product of 16 of them neither overflows nor underflows."""
    storage = O.NP_STORAGE[kind]
    if narrow and kind in ("f32", "f64"):
        return (rng.uniform(0.5, 2.0, shape) * rng.choice([-1.0, 1.0], shape)).astype(storage)
    if kind == "f32":
        return (rng.standard_normal(shape) * 10.0 ** rng.integers(-3, 4, shape)).astype(np.float32)
    if kind == "f64":
        return rng.standard_normal(shape) * 10.0 ** rng.integers(-6, 7, shape)
    if kind in ("bf16", "f16"):
        # 16-bit patterns with the top exponent bit clear: every magnitude is below 2, so neither the
        # inputs nor a sum or product of 16 of them is Inf or NaN
        return (rng.integers(0, 1 << 16, shape, dtype=np.uint32) & 0xBFFF).astype(np.uint16)
    info = np.iinfo(storage)
    return rng.integers(info.min, int(info.max) + 1, shape, dtype=storage)


def _count(rng, limit):
    """Log-uniform in [1, limit], with the small end and exact powers of two over-represented."""
    n = int(2 ** rng.uniform(0, np.log2(limit)))
    if rng.random() < 0.3:
        n = 1 << int(np.log2(n))
    return max(1, min(limit, n))


@pytest.mark.parametrize("npes,seed", [(4, 101), (5, 105), (8, 102), (12, 103), (16, 104), (33, 107), (64, 106)])
def test_random_collectives_on_random_teams(npes, seed):
    seed += SEED_OFFSET
    rng = np.random.default_rng(seed)
    world = (0, 1, npes)
    with runtime(npes, 4 * (CAP + 2 * GUARD) + (4 << 20)) as rt:
        src = rt.malloc(CAP + 2 * GUARD); dst = rt.malloc(CAP + 2 * GUARD)
        for case in range(150):
            # a random strided team (or the world team)
            if rng.random() < 0.3:
                team, triple = N.TEAM_WORLD, world
            else:
                size = int(rng.integers(1, npes + 1))
                stride = int(rng.integers(1, max(2, (npes - 1) // max(1, size - 1) + 1))) if size > 1 else 1
                start = int(rng.integers(0, npes - (size - 1) * stride))
                team = rt.team_split_strided(N.TEAM_WORLD, start, stride, size)
                triple = O.team_split_strided(world, npes, start, stride, size)
            members = O.team_members(triple)
            size = len(members)
            outside = [pe for pe in range(npes) if pe not in members]
            what = ("reduce", "reducescatter", "fcollect", "alltoall", "broadcast")[int(rng.integers(0, 5))]
            op = None
            tname = REDUCE_TYPES_STANDARD[int(rng.integers(0, len(REDUCE_TYPES_STANDARD)))]
            storage, kind = RMA_TYPES[tname]
            es = np.dtype(storage).itemsize
            if what in ("reduce", "reducescatter"):
                ops = ["and", "or", "xor", "min", "max", "sum", "prod"] if tname in REDUCE_TYPES_BITWISE else ["min", "max", "sum", "prod"]
                op = ops[int(rng.integers(0, len(ops)))]
            per = CAP // (size if what != "reduce" and what != "broadcast" else 1) // es
            n = _count(rng, max(1, min(per, 60000)))
            soff = int(rng.integers(0, GUARD // es)) * es
            doff = int(rng.integers(0, GUARD // es)) * es
            if what in ("fcollect", "alltoall", "broadcast") and rng.random() < 0.5:
                tname, storage, kind, es = None, np.uint8, "u8", 1       # the untyped *mem form, any byte offset
                n = _count(rng, max(1, min(CAP // size, 200000)))
                soff = int(rng.integers(0, GUARD)); doff = int(rng.integers(0, GUARD))
            src_elems = n * (size if what in ("reducescatter", "alltoall") else 1)
            dst_elems = n * (size if what in ("fcollect", "alltoall") else 1)
            data = _random_values(rng, kind, (npes, src_elems), narrow=what in ("reduce", "reducescatter") and op == "prod")
            rt.fill(dst, 0xCD, CAP + 2 * GUARD)
            rt.upload_all(src, data, soff)
            root = int(rng.integers(0, size))
            note("case %d/%d: npes=%d team=%s %s %s n=%d soff=%d doff=%d root=%d"
                 % (seed, case, npes, triple, what, tname or "mem", n, soff, doff, root))
            rows = data[members]
            if what == "reduce":
                rt.reduce(tname, op, dst + doff, src + soff, n, team=team)
                want = np.broadcast_to(O.reduce(kind, op, rows), (size, n))
            elif what == "reducescatter":
                rt.reducescatter(tname, op, dst + doff, src + soff, n, team=team)
                want = O.reducescatter(kind, op, rows)
            elif what == "fcollect":
                if tname: rt.fcollect(tname, dst + doff, src + soff, n, team=team)
                else: rt.fcollectmem(dst + doff, src + soff, n, team=team)
                want = O.fcollect(rows.view(np.uint8)).view(storage)
            elif what == "alltoall":
                if tname: rt.alltoall(tname, dst + doff, src + soff, n, team=team)
                else: rt.alltoallmem(dst + doff, src + soff, n, team=team)
                want = O.alltoall(rows.view(np.uint8)).view(storage)
            else:
                if tname: rt.broadcast(tname, dst + doff, src + soff, n, root, team=team)
                else: rt.broadcastmem(dst + doff, src + soff, n, root, team=team)
                want = np.broadcast_to(rows[root], (size, n))
            rt.sync()
            whole = rt.download_all(dst, (CAP + 2 * GUARD,), np.uint8)
            lo, hi = doff, doff + dst_elems * es
            for i, pe in enumerate(members):
                got = whole[pe, lo:hi].view(storage)
                assert bits_equal(got, np.ascontiguousarray(want[i])), (case, what, tname, pe)
                assert (whole[pe, :lo] == 0xCD).all() and (whole[pe, hi:] == 0xCD).all(), (case, "wrote outside", pe)
            for pe in outside:
                assert (whole[pe] == 0xCD).all(), (case, "touched a PE outside the team", pe)
            if team != N.TEAM_WORLD:
                rt.team_destroy(team)
        rt.free(src); rt.free(dst)


@pytest.mark.parametrize("npes,seed", [(6, 201), (8, 202), (16, 203)])
def test_random_in_kernel_collectives(npes, seed):
    seed += SEED_OFFSET
    """The same collectives called from inside a kernel (one block per PE) in a random scope with a
    random block size: float sum reduce / reducescatter and the untyped copies, sizes on both sides of
    the packet path's limit."""
    rng = np.random.default_rng(seed)
    world = (0, 1, npes)
    cap = 1 << 18
    with runtime(npes, 4 * (cap + 2 * GUARD) + (4 << 20)) as rt:
        perf = rt.perftest()
        src = rt.malloc(cap + 2 * GUARD); dst = rt.malloc(cap + 2 * GUARD)
        for case in range(120):
            if rng.random() < 0.4:
                team, triple = N.TEAM_WORLD, world
            else:
                size = int(rng.integers(1, npes + 1))
                stride = int(rng.integers(1, max(2, (npes - 1) // max(1, size - 1) + 1))) if size > 1 else 1
                start = int(rng.integers(0, npes - (size - 1) * stride))
                team = rt.team_split_strided(N.TEAM_WORLD, start, stride, size)
                triple = O.team_split_strided(world, npes, start, stride, size)
            members = O.team_members(triple)
            size = len(members)
            outside = [pe for pe in range(npes) if pe not in members]
            what = int(rng.integers(0, 5))       # reduce, reducescatter, fcollectmem, alltoallmem, broadcastmem
            scope = (N.SCOPE_THREAD, N.SCOPE_WARP, N.SCOPE_BLOCK)[int(rng.integers(0, 3))]
            threads = (64, 128, 256, 512, 1024)[int(rng.integers(0, 5))]
            es = 4 if what <= 1 else 1
            per_member = what in (1, 2, 3)
            n = _count(rng, max(1, min(cap // (size if per_member else 1) // es, 3000 if scope == N.SCOPE_THREAD else 40000)))
            soff = int(rng.integers(0, GUARD // es)) * es
            doff = int(rng.integers(0, GUARD // es)) * es
            src_elems = n * (size if what in (1, 3) else 1)
            dst_elems = n * (size if what in (2, 3) else 1)
            if es == 4:
                data = _random_values(rng, "f32", (npes, src_elems))
            else:
                data = _random_values(rng, "u8", (npes, src_elems))
            root = int(rng.integers(0, size))
            rt.fill(dst, 0xCD, cap + 2 * GUARD)
            rt.upload_all(src, data, soff)
            note("case %d/%d: npes=%d team=%s what=%d scope=%d threads=%d n=%d soff=%d doff=%d root=%d"
                 % (seed, case, npes, triple, what, scope, threads, n, soff, doff, root))
            assert perf.nvshmem_perftest_device_team_coll(what, team, dst + doff, src + soff, n, root, scope, threads, None) == 0
            rt.sync()
            rows = data[members]
            if what == 0:
                want = np.broadcast_to(O.reduce("f32", "sum", rows), (size, n))
            elif what == 1:
                want = O.reducescatter("f32", "sum", rows)
            elif what == 2:
                want = O.fcollect(rows)
            elif what == 3:
                want = O.alltoall(rows)
            else:
                want = np.broadcast_to(rows[root], (size, n))
            whole = rt.download_all(dst, (cap + 2 * GUARD,), np.uint8)
            lo, hi = doff, doff + dst_elems * es
            for i, pe in enumerate(members):
                got = whole[pe, lo:hi].view(np.float32 if es == 4 else np.uint8)
                assert bits_equal(got, np.ascontiguousarray(want[i])), (case, what, pe)
                assert (whole[pe, :lo] == 0xCD).all() and (whole[pe, hi:] == 0xCD).all(), (case, "wrote outside", pe)
            for pe in outside:
                assert (whole[pe] == 0xCD).all(), (case, "touched a PE outside the team", pe)
            flag, rec = rt.read_timeout(0)
            assert flag == 0, rec
            if team != N.TEAM_WORLD:
                rt.team_destroy(team)
        rt.free(src); rt.free(dst)


@pytest.mark.parametrize("scope,threads", [(N.SCOPE_WARP, 64), (N.SCOPE_BLOCK, 256), (N.SCOPE_BLOCK, 1024),
                                           (N.SCOPE_THREAD, 64)])
def test_large_in_kernel_pushes(scope, threads):
    """In-kernel fcollect / alltoall / broadcast from 32 KiB to 256 KiB per member: a common source is
    fanned out at any size, different sources up to 32 KiB each, beyond that a copy per member; with
    and without a common offset of source and dest within 16 bytes.  Broadcasts of this length are
    fetched by every PE between two barriers instead of pushed by the root."""
    npes = 8
    rng = np.random.default_rng(300 + threads)
    top = (256 << 10) + 48
    with runtime(npes, 10 * npes * top + (16 << 20)) as rt:
        perf = rt.perftest()
        src = rt.malloc(npes * top + 64); dst = rt.malloc(npes * top + 64)
        for nbytes in (32768, 32784, 100003, top):
            for soff, doff in ((0, 0), (5, 21), (3, 5)):
                data = rng.integers(0, 256, (npes, npes * nbytes), dtype=np.uint8)
                rt.upload_all(src, data, soff)
                for what in (2, 3, 4):
                    rt.fill(dst, 0xCD, npes * top + 64)
                    note("large push what=%d bytes=%d soff=%d doff=%d scope=%d threads=%d" % (what, nbytes, soff, doff, scope, threads))
                    assert perf.nvshmem_perftest_device_team_coll(what, N.TEAM_WORLD, dst + doff, src + soff, nbytes, 5,
                                                                  scope, threads, None) == 0
                    rt.sync()
                    out_bytes = nbytes if what == 4 else npes * nbytes
                    got = rt.download_all(dst, (npes * top + 64,), np.uint8)
                    if what == 2:
                        want = O.fcollect(data[:, :nbytes])
                    elif what == 3:
                        want = O.alltoall(data)
                    else:
                        want = np.broadcast_to(data[5, :nbytes], (npes, nbytes))
                    assert np.array_equal(got[:, doff:doff + out_bytes], want), (what, nbytes, soff, doff)
                    assert (got[:, :doff] == 0xCD).all() and (got[:, doff + out_bytes:] == 0xCD).all()
        flag, rec = rt.read_timeout(0)
        assert flag == 0, rec
        rt.free(src); rt.free(dst)
