"""GPU parity of teams through the C ABI: the team table against the oracle's team arithmetic (host
queries and the same queries evaluated in device code), host-launched collectives on strided teams
and on the row / column families of a 2-D split (every team of the family in one call, PEs outside
untouched), the in-kernel collectives and the team barrier in all scopes, and handle reuse."""
import ctypes as C

import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import bits_equal, note, runtime

pytestmark = pytest.mark.gpu

NPES = 16
WORLD = (0, 1, NPES)


@pytest.fixture(scope="module")
def rt():
    with runtime(NPES, 1 << 24) as r:
        yield r


def _views(rt, team):
    return [rt.team_view(team, pe) for pe in range(rt.npes)]


def _expect_views(members_of):
    """members_of[pe] = (start, stride, size) or None -> the view tuples the library must hold."""
    out = []
    for pe, t in enumerate(members_of):
        if t is None:
            out.append(None)
        else:
            out.append((t[0], t[1], t[2], O.team_members(t).index(pe)))
    return out


def _check_views(rt, team, members_of):
    for pe, (got, want) in enumerate(zip(_views(rt, team), _expect_views(members_of))):
        if want is None:
            assert got[2] == 0, (team, pe, got)
        else:
            assert got == want, (team, pe, got, want)


def _groups(members_of):
    seen = []
    for t in members_of:
        if t is not None and t not in seen:
            seen.append(t)
    return seen


# ---------------------------------------------------------------------------------------------
# the table
# ---------------------------------------------------------------------------------------------
def test_predefined_teams(rt):
    for team in (N.TEAM_WORLD, 1, 2, 4):       # WORLD, SHARED, NODE, SAME_GPU: everybody
        _check_views(rt, team, [WORLD] * NPES)
        assert rt.lib.nvshmem_team_n_pes(team) == NPES and rt.lib.nvshmem_team_my_pe(team) == 0
    _check_views(rt, 3, [(pe, 1, 1) for pe in range(NPES)])      # SAME_MYPE_NODE: each PE alone
    _check_views(rt, 5, [(0, 1, 1)] + [None] * (NPES - 1))       # GPU_LEADERS: PE 0
    assert rt.lib.nvshmem_team_n_pes(-1) == -1 and rt.lib.nvshmem_team_my_pe(-1) == -1
    assert rt.lib.nvshmem_team_n_pes(17) == -1
    rt.team_destroy(N.TEAM_WORLD)               # refused, the team stays
    assert "pre-defined" in rt.last_error()
    assert rt.lib.nvshmem_team_n_pes(N.TEAM_WORLD) == NPES


def test_split_strided_matches_the_oracle_and_rejects_what_the_reference_rejects(rt):
    made = []
    for start, stride, size in ((0, 1, 16), (0, 2, 8), (1, 2, 8), (4, 3, 4), (15, 1, 1), (2, 6, 3)):
        want = O.team_split_strided(WORLD, NPES, start, stride, size)
        assert want is not None
        note("split_strided WORLD %d %d %d" % (start, stride, size))
        t = rt.team_split_strided(N.TEAM_WORLD, start, stride, size)
        made.append(t)
        assert t >= 6
        members = O.team_members(want)
        _check_views(rt, t, [want if pe in members else None for pe in range(NPES)])
        # a split of the split: indices count the parent's members
        for s2, st2, sz2 in ((0, 1, size), (size - 1, 1, 1), (0, 2, (size + 1) // 2), (1, 3, 2)):
            child = O.team_split_strided(want, NPES, s2, st2, sz2)
            if child is None:
                with pytest.raises(N.host.NvshmemError, match="invalid <start, stride, size>"):
                    rt.team_split_strided(t, s2, st2, sz2)
                continue
            t2 = rt.team_split_strided(t, s2, st2, sz2)
            cm = O.team_members(child)
            _check_views(rt, t2, [child if pe in cm else None for pe in range(NPES)])
            # translate between parent, child and WORLD as PE 0 sees them (host answers for PE 0)
            if 0 in members:
                for i in range(size + 2):
                    assert rt.lib.nvshmem_team_translate_pe(t, i, N.TEAM_WORLD) == \
                        O.team_translate_pe(want, i, WORLD)
                    if 0 in cm:
                        assert rt.lib.nvshmem_team_translate_pe(t, i, t2) == O.team_translate_pe(want, i, child)
            rt.team_destroy(t2)
    for bad in ((-1, 1, 4), (16, 1, 1), (0, 0, 4), (0, 1, 0), (0, 1, 17), (8, 2, 5), (0, 16, 2)):
        assert O.team_split_strided(WORLD, NPES, *bad) is None
        with pytest.raises(N.host.NvshmemError, match="invalid <start, stride, size>"):
            rt.team_split_strided(N.TEAM_WORLD, *bad)
    t = C.c_int32(5)
    assert rt.lib.nvshmem_team_split_strided(-1, 0, 1, 4, None, 0, C.byref(t)) != 0 and t.value == -1
    for t in made:
        rt.team_destroy(t)


@pytest.mark.parametrize("xrange_", [4, 5, 16, 1, 40])
def test_split_2d_rows_and_columns(rt, xrange_):
    note("split_2d xrange=%d" % xrange_)
    x, y = rt.team_split_2d(N.TEAM_WORLD, xrange_)
    want = [O.team_split_2d(WORLD, xrange_, pe) for pe in range(NPES)]
    _check_views(rt, x, [w[0] for w in want])
    _check_views(rt, y, [w[1] for w in want])
    # host queries answer for PE 0
    assert rt.lib.nvshmem_team_n_pes(x) == want[0][0][2] and rt.lib.nvshmem_team_my_pe(y) == 0
    # the same queries in device code, for every PE
    perf = rt.perftest()
    out = rt.calloc(4 + 64, 4)
    assert perf.nvshmem_perftest_team_query(out, x, y, None) == 0
    rt.sync()
    got = rt.download_all(out, (4 + 64,), np.int32)
    for pe in range(NPES):
        xt, yt = want[pe]
        assert got[pe, 0] == O.team_members(xt).index(pe) and got[pe, 1] == xt[2]
        assert got[pe, 2] == O.team_members(yt).index(pe) and got[pe, 3] == yt[2]
        for i in range(64):
            assert got[pe, 4 + i] == O.team_translate_pe(xt, i, yt), (pe, i)
    rt.free(out)
    rt.team_destroy(x); rt.team_destroy(y)


def test_handles_are_reused_and_run_out(rt):
    first = rt.team_split_strided(N.TEAM_WORLD, 0, 1, 4)
    rt.team_destroy(first)
    made = []
    while True:
        t = C.c_int32(-1)
        rc = rt.lib.nvshmem_team_split_strided(N.TEAM_WORLD, 0, 1, 4, None, 0, C.byref(t))
        if rc != 0:
            assert t.value == -1 and "in use" in rt.last_error()
            break
        made.append(t.value)
    assert made[0] == first and len(made) == 32 - 6 and sorted(set(made)) == made
    cfg = (C.c_int32 * 16)()
    rt.lib.nvshmem_team_get_config(made[3], cfg)
    assert cfg[1] == -1                              # num_contexts of the default configuration
    for t in made:
        rt.team_destroy(t)
    rt.team_destroy(made[0])
    assert "does not exist" in rt.last_error()


# ---------------------------------------------------------------------------------------------
# host-launched collectives on teams
# ---------------------------------------------------------------------------------------------
def _member_rows(data, team):
    return data[O.team_members(team)]


def _run_host_collectives(rt, team, members_of, n, rng):
    """Every collective once on `team`; members_of[pe] is the oracle's triple for PE pe (or None)."""
    groups = _groups(members_of)
    max_size = max(g[2] for g in groups)
    src = rt.malloc(max_size * n * 4 + 64); dst = rt.malloc(max_size * n * 4 + 64)
    outside = [pe for pe in range(rt.npes) if members_of[pe] is None]

    def fresh(shape_elems):
        data = (rng.standard_normal((rt.npes, shape_elems)) * 10.0 ** rng.integers(-3, 4, (rt.npes, shape_elems))).astype(np.float32)
        rt.fill(dst, 0xCD, max_size * n * 4 + 64)
        rt.upload_all(src, data)
        return data

    def untouched(nelems):
        for pe in outside:
            assert (rt.download(dst, pe, (nelems,), np.uint32) == 0xCDCDCDCD).all(), pe

    data = fresh(n)
    note("team %d reduce float sum n=%d" % (team, n))
    rt.reduce("float", "sum", dst, src, n, team=team)
    for g in groups:
        want = O.reduce("f32", "sum", _member_rows(data, g))
        for pe in O.team_members(g):
            assert bits_equal(rt.download(dst, pe, (n,), np.float32), want), (g, pe)
    untouched(n)
    # in place and the element-at-a-time kernel
    rt.reduce("float", "max", src + 4, src + 4, n - 1, team=team)
    for g in groups:
        want = O.reduce("f32", "max", _member_rows(data, g)[:, 1:])
        assert bits_equal(rt.download(src, O.team_members(g)[-1], (n - 1,), np.float32, 4), want), g
    for pe in outside:
        assert bits_equal(rt.download(src, pe, (n,), np.float32), data[pe])

    data = fresh(max_size * n)
    note("team %d reducescatter float sum n=%d" % (team, n))
    rt.reducescatter("float", "sum", dst, src, n, team=team)
    for g in groups:
        rows = _member_rows(data, g)[:, :g[2] * n]
        want = O.reducescatter("f32", "sum", rows)
        for i, pe in enumerate(O.team_members(g)):
            assert bits_equal(rt.download(dst, pe, (n,), np.float32), want[i]), (g, pe)
    untouched(n)

    data = fresh(max_size * n)
    raw = data.view(np.uint8)
    note("team %d fcollect / alltoall / broadcast" % team)
    rt.fcollectmem(dst, src, n * 4 - 3, team=team)
    for g in groups:
        want = O.fcollect(_member_rows(raw, g)[:, :n * 4 - 3])
        for i, pe in enumerate(O.team_members(g)):
            assert np.array_equal(rt.download(dst, pe, (g[2] * (n * 4 - 3),), np.uint8), want[i]), (g, pe)
    untouched(n)
    rt.fill(dst, 0xCD, max_size * n * 4 + 64)
    rt.alltoallmem(dst + 1, src + 2, n * 4 - 5, team=team)
    for g in groups:
        want = O.alltoall(_member_rows(raw, g)[:, 2:2 + g[2] * (n * 4 - 5)])
        for i, pe in enumerate(O.team_members(g)):
            assert np.array_equal(rt.download(dst, pe, (g[2] * (n * 4 - 5),), np.uint8, 1), want[i]), (g, pe)
    untouched(n)
    rt.fill(dst, 0xCD, max_size * n * 4 + 64)
    root = min(g[2] for g in groups) - 1
    rt.broadcastmem(dst, src, n * 4 - 1, root, team=team)
    for g in groups:
        want = raw[O.team_members(g)[root], :n * 4 - 1]
        for pe in O.team_members(g):
            assert np.array_equal(rt.download(dst, pe, (n * 4 - 1,), np.uint8), want), (g, pe)
    untouched(n)
    with pytest.raises(N.host.NvshmemError, match="root"):
        rt.broadcastmem(dst, src, 16, root + 1, team=team)
    rt.free(src); rt.free(dst)


@pytest.mark.parametrize("start,stride,size", [(0, 1, 8), (1, 2, 8), (3, 4, 3), (0, 1, 16), (5, 1, 1)])
def test_host_collectives_on_a_strided_team(rt, start, stride, size):
    rng = np.random.default_rng(start * 100 + stride * 10 + size)
    t = rt.team_split_strided(N.TEAM_WORLD, start, stride, size)
    triple = O.team_split_strided(WORLD, NPES, start, stride, size)
    members = O.team_members(triple)
    _run_host_collectives(rt, t, [triple if pe in members else None for pe in range(NPES)], 2052, rng)
    rt.team_destroy(t)


@pytest.mark.parametrize("xrange_", [8, 4, 5])
def test_host_collectives_on_rows_and_columns(rt, xrange_):
    rng = np.random.default_rng(xrange_)
    x, y = rt.team_split_2d(N.TEAM_WORLD, xrange_)
    want = [O.team_split_2d(WORLD, xrange_, pe) for pe in range(NPES)]
    _run_host_collectives(rt, x, [w[0] for w in want], 1028, rng)     # xrange 5: ragged last row
    _run_host_collectives(rt, y, [w[1] for w in want], 1028, rng)
    # rows of 8 take the kernel specialised for 8 members; a sub-split of every row at once
    half = rt.team_split_strided(x, 0, 2, (min(xrange_, NPES) + 1) // 2) if xrange_ != 5 else None
    if half is not None:
        triples = [O.team_split_strided(w[0], NPES, 0, 2, (xrange_ + 1) // 2) for w in want]
        mo = [t if pe in O.team_members(t) else None for pe, t in enumerate(triples)]
        _check_views(rt, half, mo)
        _run_host_collectives(rt, half, mo, 516, rng)
        rt.team_destroy(half)
    rt.team_destroy(x); rt.team_destroy(y)


def test_team_argument_errors(rt):
    a = rt.malloc(4096); b = rt.malloc(4096)
    with pytest.raises(N.host.NvshmemError, match="does not exist"):
        rt.reduce("float", "sum", a, b, 16, team=9)
    with pytest.raises(N.host.NvshmemError, match="does not exist"):
        rt.fcollectmem(a, b, 16, team=-1)
    assert rt.lib.nvshmem_team_sync(11) != 0 and rt.lib.nvshmem_team_sync(N.TEAM_WORLD) == 0
    assert rt.lib.nvshmemx_barrier_on_stream(2, None) == 0
    rt.free(a); rt.free(b)


# ---------------------------------------------------------------------------------------------
# in-kernel collectives and barriers on teams
# ---------------------------------------------------------------------------------------------
# n = 517: copy-and-barrier paths; n = 12: the packet paths (one packet per lane) on every team
@pytest.mark.parametrize("n", [517, 12])
@pytest.mark.parametrize("scope,threads", [(N.SCOPE_THREAD, 64), (N.SCOPE_WARP, 128), (N.SCOPE_BLOCK, 256)])
def test_device_scope_collectives_on_teams(rt, scope, threads, n):
    perf = rt.perftest()
    rng = np.random.default_rng(50 + scope + n)
    x, y = rt.team_split_2d(N.TEAM_WORLD, 4)
    odd = rt.team_split_strided(N.TEAM_WORLD, 1, 2, 8)
    want2d = [O.team_split_2d(WORLD, 4, pe) for pe in range(NPES)]
    odd_t = (1, 2, 8)
    cases = [(x, [w[0] for w in want2d]), (y, [w[1] for w in want2d]),
             (odd, [odd_t if pe % 2 else None for pe in range(NPES)])]
    src = rt.malloc(8 * n * 4 + 64); dst = rt.malloc(8 * n * 4 + 64)
    for team, members_of in cases:
        groups = _groups(members_of)
        size = groups[0][2]
        outside = [pe for pe in range(NPES) if members_of[pe] is None]

        def run(what, count, root=0):
            rt.fill(dst, 0xCD, 8 * n * 4 + 64)
            note("device team coll what=%d team=%d scope=%d" % (what, team, scope))
            assert perf.nvshmem_perftest_device_team_coll(what, team, dst, src, count, root, scope,
                                                          threads, None) == 0
            rt.sync()
            for pe in outside:
                assert (rt.download(dst, pe, (n,), np.uint32) == 0xCDCDCDCD).all()

        data = rng.standard_normal((NPES, size * n)).astype(np.float32)
        raw = data.view(np.uint8)
        rt.upload_all(src, data)
        run(0, n)
        for g in groups:
            want = O.reduce("f32", "sum", _member_rows(data, g)[:, :n])
            for pe in O.team_members(g):
                assert bits_equal(rt.download(dst, pe, (n,), np.float32), want), (team, g, pe)
        run(1, n)
        for g in groups:
            want = O.reducescatter("f32", "sum", _member_rows(data, g))
            for i, pe in enumerate(O.team_members(g)):
                assert bits_equal(rt.download(dst, pe, (n,), np.float32), want[i]), (team, g, pe)
        run(2, n * 4 - 3)
        for g in groups:
            want = O.fcollect(_member_rows(raw, g)[:, :n * 4 - 3])
            for i, pe in enumerate(O.team_members(g)):
                assert np.array_equal(rt.download(dst, pe, (size * (n * 4 - 3),), np.uint8), want[i])
        run(3, n * 4 - 3)
        for g in groups:
            want = O.alltoall(_member_rows(raw, g)[:, :size * (n * 4 - 3)])
            for i, pe in enumerate(O.team_members(g)):
                assert np.array_equal(rt.download(dst, pe, (size * (n * 4 - 3),), np.uint8), want[i])
        run(4, n * 4 - 3, root=size - 1)
        for g in groups:
            want = raw[O.team_members(g)[size - 1], :n * 4 - 3]
            for pe in O.team_members(g):
                assert np.array_equal(rt.download(dst, pe, (n * 4 - 3,), np.uint8), want)
        # barriers among the members only
        counter = rt.calloc(1, 8); errors = rt.calloc(1, 8)
        assert perf.nvshmem_perftest_device_team_barrier(counter, errors, 50, team, scope, threads, None) == 0
        rt.sync()
        got = rt.download_all(errors, (1,), np.uint64)
        cnt = rt.download_all(counter, (1,), np.uint64)
        assert (got == 0).all()
        for pe in range(NPES):
            assert cnt[pe, 0] == (0 if pe in outside else 50)
        flag, rec = rt.read_timeout(0)
        assert flag == 0, rec
        rt.free(counter); rt.free(errors)
    rt.free(src); rt.free(dst)
    for t in (x, y, odd):
        rt.team_destroy(t)


def test_warpgroup_barrier_on_world_and_strided_teams(rt):
    """nvshmemx_barrier_warpgroup: one group of up to 256 threads of every member's block runs the
    barrier rounds while the block's other threads have left; first, middle and short last group."""
    perf = rt.perftest()
    odd = rt.team_split_strided(N.TEAM_WORLD, 1, 2, NPES // 2)
    for team, members in ((N.TEAM_WORLD, list(range(NPES))), (odd, list(range(1, NPES, 2)))):
        for threads, group in ((256, 0), (512, 1), (768, 1), (640, 2), (1024, 3), (64, 0)):
            note("warpgroup barrier team=%d threads=%d group=%d" % (team, threads, group))
            counter = rt.calloc(1, 8); errors = rt.calloc(1, 8)
            assert perf.nvshmem_perftest_device_warpgroup_barrier(counter, errors, 40, team, group, threads, None) == 0
            rt.sync()
            assert (rt.download_all(errors, (1,), np.uint64) == 0).all()
            cnt = rt.download_all(counter, (1,), np.uint64)
            for pe in range(NPES):
                assert cnt[pe, 0] == (40 if pe in members else 0)
            flag, rec = rt.read_timeout(0)
            assert flag == 0, rec
            rt.free(counter); rt.free(errors)
    counter = rt.calloc(1, 8); errors = rt.calloc(1, 8)
    assert perf.nvshmem_perftest_device_warpgroup_barrier(counter, errors, 1, N.TEAM_WORLD, 2, 512, None) != 0
    rt.free(counter); rt.free(errors)
    rt.team_destroy(odd)


def test_maxloc_reduce_and_device_identification(rt):
    """nvshmemx_double2_maxloc_reduce_block on the world team, a strided team and the rows of a 2-D
    split, with ties and NaNs in the values; plus what the device-side identification calls report."""
    perf = rt.perftest()
    rng = np.random.default_rng(61)
    x, y = rt.team_split_2d(N.TEAM_WORLD, 4)
    odd = rt.team_split_strided(N.TEAM_WORLD, 1, 2, 8)
    want2d = [O.team_split_2d(WORLD, 4, pe) for pe in range(NPES)]
    cases = [(N.TEAM_WORLD, [WORLD] * NPES), (x, [w[0] for w in want2d]),
             (odd, [(1, 2, 8) if pe % 2 else None for pe in range(NPES)])]
    nmax = 70
    src = rt.malloc(nmax * 16); dst = rt.malloc(nmax * 16); info = rt.calloc(4, 4)
    for team, members_of in cases:
        for n, threads in ((1, 64), (nmax, 256)):
            pairs = np.empty((NPES, n, 2))
            pairs[:, :, 0] = rng.integers(-3, 4, (NPES, n))          # few distinct values: many ties
            pairs[:, :, 1] = np.arange(NPES)[:, None] * 1000 + np.arange(n)[None, :]
            pairs[rng.random((NPES, n)) < 0.1, 0] = np.nan
            rt.upload_all(src, pairs)
            rt.fill(dst, 0xCD, nmax * 16)
            note("maxloc team=%d n=%d threads=%d" % (team, n, threads))
            assert perf.nvshmem_perftest_device_maxloc(team, dst, src, n, 2, threads, info, None) == 0
            rt.sync()
            for g in _groups(members_of):
                members = O.team_members(g)
                want = O.maxloc_reduce(pairs[members])
                for i, pe in enumerate(members):
                    assert bits_equal(rt.download(dst, pe, (n, 2), np.float64), want[i]), (team, g, pe, n)
            for pe in range(NPES):
                if members_of[pe] is None:
                    assert (rt.download(dst, pe, (n * 4,), np.uint32) == 0xCDCDCDCD).all()
    got = rt.download_all(info, (4,), np.int32)
    name = C.create_string_buffer(256)
    rt.lib.nvshmem_info_get_name(name)
    assert (got == np.array([1, 3, 30501, len(name.value)], np.int32)).all(), got
    assert perf.nvshmem_perftest_device_maxloc(N.TEAM_WORLD, dst, src, 1 << 40, 1, 64, None, None) != 0
    rt.team_destroy(x); rt.team_destroy(y); rt.team_destroy(odd)
    for p in (src, dst, info):
        rt.free(p)


def test_a_reused_handle_starts_clean(rt):
    """Packet flags and barrier epochs restart when a handle is reused by other members."""
    perf = rt.perftest()
    rng = np.random.default_rng(77)
    n = 8
    src = rt.malloc(4096); dst = rt.malloc(4096)
    for round_, (start, stride, size) in enumerate(((0, 1, 4), (2, 3, 5), (1, 1, 15), (0, 2, 8))):
        t = rt.team_split_strided(N.TEAM_WORLD, start, stride, size)
        assert t == 6                                  # always the same, lowest free handle
        members = [start + i * stride for i in range(size)]
        for rep in range(3 + round_):                  # a different number of calls per life
            data = rng.standard_normal((NPES, n)).astype(np.float32)
            rt.upload_all(src, data)
            rt.fill(dst, 0xCD, 4096)
            note("reused handle round=%d rep=%d" % (round_, rep))
            assert perf.nvshmem_perftest_device_team_coll(0, t, dst, src, n, 0, N.SCOPE_BLOCK, 256, None) == 0
            rt.sync()
            want = O.reduce("f32", "sum", data[members])
            for pe in range(NPES):
                got = rt.download(dst, pe, (n,), np.float32)
                if pe in members:
                    assert bits_equal(got, want), (round_, rep, pe)
                else:
                    assert (got.view(np.uint32) == 0xCDCDCDCD).all()
            root = rep % size
            assert perf.nvshmem_perftest_device_team_coll(4, t, dst, src, n * 4, root, N.SCOPE_WARP, 64, None) == 0
            rt.sync()
            for pe in members:
                assert bits_equal(rt.download(dst, pe, (n,), np.float32), data[members[root]])
        counter = rt.calloc(1, 8); errors = rt.calloc(1, 8)
        assert perf.nvshmem_perftest_device_team_barrier(counter, errors, 5 + round_, t, N.SCOPE_BLOCK, 128, None) == 0
        rt.sync()
        assert (rt.download_all(errors, (1,), np.uint64) == 0).all()
        rt.free(counter); rt.free(errors)
        rt.team_destroy(t)
    assert rt.read_timeout(0)[0] == 0
    rt.free(src); rt.free(dst)
