"""Pins the CPU oracle before anything is compared against it.

The reference ships no golden data for this path; what it holds are four closed-form checks in its
examples.  Those are reproduced first; the rest is pinned against independent implementations
(numpy / torch CPU arithmetic in the element type, brute-force index maps written from the
operator definitions, hand-evaluated NaN / signed-zero cases), chosen so that a wrong fold order,
swapped operands, a transposed index or a missing rounding step fails.
"""
import itertools

import numpy as np
import pytest

import oracle_lib as O

INT_KINDS = ["i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64"]


# ---------------------------------------------------------------------------------------------
# the reference's own known answers
# ---------------------------------------------------------------------------------------------
def test_kat_put_block_ring():
    # examples/put-block.cu:39,93-104: every PE sends its own rank to (mype+1)%npes;
    # the receiver must hold (mype-1+npes)%npes
    for npes in (2, 3, 8, 16):
        msg = np.repeat(np.arange(npes, dtype=np.int32)[:, None], 32, axis=1)
        got = O.ring_put(msg.view(np.uint8)).view(np.int32)
        for pe in range(npes):
            assert (got[pe] == (pe - 1 + npes) % npes).all()


@pytest.mark.parametrize("npes", [2, 4, 8])
def test_kat_allreduce_i_times_npes(npes):
    # examples/ring-reduce.cu:209,242-248 and examples/user-buffer.cu:141-152:
    # src[i] = i on every PE, sum => dst[i] = i * npes (int and float)
    n = 4096
    src_i = np.tile(np.arange(n, dtype=np.int32), (npes, 1))
    assert (O.reduce("i32", "sum", src_i) == np.arange(n) * npes).all()
    src_f = src_i.astype(np.float32)
    assert (O.reduce("f32", "sum", src_f) == (np.arange(n) * npes).astype(np.float32)).all()


# ---------------------------------------------------------------------------------------------
# integer reductions: order-free closed forms via numpy
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("kind", INT_KINDS)
@pytest.mark.parametrize("npes", [1, 2, 5, 8])
def test_integer_reduce_matches_numpy(kind, npes):
    rng = np.random.default_rng(hash((kind, npes)) % 2**32)
    dt = O.NP_STORAGE[kind]
    info = np.iinfo(dt)
    src = rng.integers(info.min, info.max, size=(npes, 513), dtype=dt, endpoint=True)
    with np.errstate(over="ignore"):
        expect = {
            "and": np.bitwise_and.reduce(src, axis=0),
            "or": np.bitwise_or.reduce(src, axis=0),
            "xor": np.bitwise_xor.reduce(src, axis=0),
            "min": src.min(axis=0),
            "max": src.max(axis=0),
            "sum": np.add.reduce(src, axis=0, dtype=dt),    # wraps modulo 2^bits
            "prod": np.multiply.reduce(src, axis=0, dtype=dt),
        }
    for op, want in expect.items():
        assert np.array_equal(O.reduce(kind, op, src), want), (kind, op)


def test_xor_self_cancels_and_cfg1_bounds():
    x = O.fill("u64", 1000, 5, 0)
    assert (O.reduce("u64", "xor", np.stack([x, x, x, x])) == 0).all()
    v = O.fill_all("i32", 8, 1 << 16, 1)
    assert v.min() >= -(1 << 20) and v.max() <= (1 << 20)
    assert abs(int(v.astype(np.int64).sum(0).max())) <= 1 << 23  # the sum cannot overflow int32


def test_undefined_pairs_are_rejected():
    x = np.zeros((2, 4), np.float32)
    for op in ("and", "or", "xor"):
        with pytest.raises(ValueError):
            O.reduce("f32", op, x)


# ---------------------------------------------------------------------------------------------
# floating point: left fold in PE order, computed in the element type
# ---------------------------------------------------------------------------------------------
def _numpy_left_fold(src, fn):
    acc = src[0].copy()
    for p in range(1, src.shape[0]):
        acc = fn(acc, src[p])
    return acc


@pytest.mark.parametrize("kind,dt", [("f32", np.float32), ("f64", np.float64)])
def test_float_sum_prod_is_left_fold_in_pe_order(kind, dt):
    rng = np.random.default_rng(7)
    # magnitudes spread over many binades so that the association order changes the result
    src = (rng.standard_normal((8, 4096)) * 10.0 ** rng.integers(-6, 7, (8, 4096))).astype(dt)
    want = _numpy_left_fold(src, np.add)
    got = O.reduce(kind, "sum", src)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    reverse = _numpy_left_fold(src[::-1], np.add)
    assert not np.array_equal(reverse, want), "input does not discriminate the fold order"
    src_p = (1.0 + rng.standard_normal((8, 4096)) * 0.3).astype(dt)
    assert np.array_equal(O.reduce(kind, "prod", src_p), _numpy_left_fold(src_p, np.multiply))


def test_f32_order_sensitive_hand_case():
    # (1e8 + 1) + -1e8 = 0 in fp32 (1 is below half an ulp of 1e8), while 1e8 + (1 + -1e8) = 0 too
    # but (1e8 + -1e8) + 1 = 1: PE order 0,1,2 must give 0 for [1e8, 1, -1e8] and 1 for [1e8, -1e8, 1]
    a = np.array([[1e8], [1.0], [-1e8]], np.float32)
    b = np.array([[1e8], [-1e8], [1.0]], np.float32)
    assert O.reduce("f32", "sum", a)[0] == 0.0
    assert O.reduce("f32", "sum", b)[0] == 1.0


def _bits(x):
    return np.asarray(x, np.float32).view(np.uint32)


def test_min_max_operand_rule_nan_and_signed_zero():
    # rule (reference reduce.cuh:96-99): max(a,b) = (a > b) ? a : b, min(a,b) = (a < b) ? a : b;
    # fold: acc = op(x0, x1); acc = op(x_i, acc).  Evaluated by hand:
    nan = np.float32("nan")
    cases_max = [
        ([nan, 1, 2], 2.0),     # (nan>1)?nan:1 = 1 ; (2>1)?2:1 = 2
        ([1, nan, 2], nan),     # (1>nan)?1:nan = nan ; (2>nan)?2:nan = nan
        ([1, 2, nan], 2.0),     # 2 ; (nan>2)?nan:2 = 2
        ([0.0, -0.0], -0.0),    # (0>-0) false -> second operand
        ([-0.0, 0.0], 0.0),
        ([0.0, 0.0, -0.0], 0.0),  # acc=0.0 ; (-0.0 > 0.0) false -> acc
    ]
    for xs, want in cases_max:
        got = O.reduce("f32", "max", np.array(xs, np.float32)[:, None])[0]
        assert _bits(got) == _bits(want) or (np.isnan(want) and np.isnan(got)), (xs, got)
    cases_min = [
        ([nan, 1, 2], 1.0),     # (nan<1)?nan:1 = 1 ; (2<1)?2:1 = 1
        ([1, nan, 0], nan),     # nan ; (0<nan)?0:nan = nan
        ([3, 2, nan], 2.0),
        ([0.0, -0.0], -0.0),    # (0 < -0) false -> second
        ([-0.0, 0.0], 0.0),
    ]
    for xs, want in cases_min:
        got = O.reduce("f32", "min", np.array(xs, np.float32)[:, None])[0]
        assert _bits(got) == _bits(want) or (np.isnan(want) and np.isnan(got)), (xs, got)
    # finite data: plain min / max
    rng = np.random.default_rng(3)
    src = rng.standard_normal((8, 1000)).astype(np.float32)
    assert np.array_equal(O.reduce("f32", "max", src), src.max(0))
    assert np.array_equal(O.reduce("f32", "min", src), src.min(0))


def test_f16_conversions_exhaustive_against_numpy():
    L = O.lib()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([L.oracle_f16_to_f32(int(h)) for h in allh], np.float32)
    both_nan = np.isnan(want) & np.isnan(got)
    assert ((want.view(np.uint32) == got.view(np.uint32)) | both_nan).all()
    rng = np.random.default_rng(11)
    f = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([65504, 65519.99, 65520, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -14,
                  6.0975552e-05, 0.0, -0.0, np.inf, -np.inf], np.float32)])
    with np.errstate(over="ignore"):
        want16 = f.astype(np.float16).view(np.uint16)
    got16 = np.array([L.oracle_f32_to_f16(float(x)) for x in f], np.uint16)
    assert np.array_equal(got16, want16)


def test_bf16_conversion_and_sum_against_torch():
    torch = pytest.importorskip("torch")
    L = O.lib()
    rng = np.random.default_rng(5)
    f = (rng.standard_normal(20000) * 10.0 ** rng.integers(-20, 20, 20000)).astype(np.float32)
    f[:6] = [1.0, 1.00390625, 1.01171875, -0.0, 3.3895314e38, 2.0 ** -133]  # ties and edges
    want = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.oracle_f32_to_bf16(float(x)) for x in f], np.uint16)
    assert np.array_equal(got, want)
    # sum / prod / max fold in bf16, one rounding per step: torch CPU adds bf16 the same way
    src = O.fill_all("bf16", 8, 4096, 4)
    t = torch.from_numpy(src.view(np.int16)).view(torch.bfloat16)
    for op, fn in (("sum", torch.add), ("prod", torch.mul), ("max", torch.maximum), ("min", torch.minimum)):
        acc = t[0].clone()
        for p in range(1, 8):
            acc = fn(acc, t[p])
        want = acc.view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(O.reduce("bf16", op, src), want), op
    # and it differs from "accumulate in fp32, round once" often enough to tell the two apart
    once = torch.from_numpy(src.view(np.int16)).view(torch.bfloat16).float().sum(0).to(torch.bfloat16)
    assert (once.view(torch.int16).numpy().view(np.uint16) != O.reduce("bf16", "sum", src)).any()


def test_f16_sum_against_numpy_half_arithmetic():
    src = O.fill_all("f16", 8, 4096, 9)
    h = src.view(np.float16)
    assert np.array_equal(O.reduce("f16", "sum", src), _numpy_left_fold(h, np.add).view(np.uint16))
    assert np.array_equal(O.reduce("f16", "max", src), h.max(0).view(np.uint16))


# ---------------------------------------------------------------------------------------------
# permutations: brute force from the operator definitions
#   fcollect: dest@q[p*n + k] = src@p[k]        alltoall: dest@q[p*n + k] = src@p[q*n + k]
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("npes,seg", [(1, 5), (2, 1), (3, 7), (8, 16), (16, 3)])
def test_fcollect_alltoall_brute_force(npes, seg):
    rng = np.random.default_rng(npes * 100 + seg)
    src_f = rng.integers(0, 256, (npes, seg), dtype=np.uint8)
    got = O.fcollect(src_f)
    for q, p, k in itertools.product(range(npes), range(npes), range(seg)):
        assert got[q, p * seg + k] == src_f[p, k]
    src_a = rng.integers(0, 256, (npes, npes * seg), dtype=np.uint8)
    got = O.alltoall(src_a)
    for q, p, k in itertools.product(range(npes), range(npes), range(seg)):
        assert got[q, p * seg + k] == src_a[p, q * seg + k]
    # alltoall is an involution: exchanging twice restores the input
    assert np.array_equal(O.alltoall(got), src_a)


def test_ring_get_is_inverse_direction():
    data = O.fill_all("bytes", 5, 77, 2)
    put = O.ring_put(data)
    assert np.array_equal(O.ring_get(put), data)  # get from right neighbour undoes put to it


# ---------------------------------------------------------------------------------------------
# comparison / signal operators, nvshmem_ptr
# ---------------------------------------------------------------------------------------------
def test_compare_tables():
    import operator
    L = O.lib()
    ops = [operator.eq, operator.ne, operator.gt, operator.le, operator.lt, operator.ge]  # EQ NE GT LE LT GE
    vals = [0, 1, 2, 2**63 - 1, 2**63, 2**64 - 1]
    for cmp, fn in enumerate(ops):
        for a in vals:
            for b in vals:
                assert bool(L.oracle_compare_u64(a, cmp, b)) == fn(a, b)
    svals = [-2**63, -1, 0, 1, 2**63 - 1]
    for cmp, fn in enumerate(ops):
        for a in svals:
            for b in svals:
                assert bool(L.oracle_compare_i64(a, cmp, b)) == fn(a, b)


def test_signal_op_values():
    L = O.lib()
    assert L.oracle_signal_op(5, 9, 9) == 9          # NVSHMEM_SIGNAL_SET = 9
    assert L.oracle_signal_op(5, 9, 10) == 14        # NVSHMEM_SIGNAL_ADD = 10
    assert L.oracle_signal_op(2**64 - 1, 2, 10) == 1  # wraps
    assert L.oracle_signal_op(5, 9, 3) == 5


def test_ptr_closed_form():
    L = O.lib()
    base, size, npes = 0x7000_0000_0000, 1 << 20, 8
    assert L.oracle_ptr(base, size, npes, base + 100, 3) == base + 3 * size + 100
    assert L.oracle_ptr(base, size, npes, base + 5 * size + 100, 0) == base + 100   # any slice
    assert L.oracle_ptr(base, size, npes, base + 100, -1) == 0
    assert L.oracle_ptr(base, size, npes, base + 100, 8) == 0
    assert L.oracle_ptr(base, size, npes, base - 1, 0) == 0
    assert L.oracle_ptr(base, size, npes, base + 8 * size, 0) == 0
    assert L.oracle_ptr(base, size, npes, base + 8 * size - 1, 7) == base + 8 * size - 1


# ---------------------------------------------------------------------------------------------
# input generators
# ---------------------------------------------------------------------------------------------
def test_splitmix64_reference_vector():
    # SplitMix64 (Steele, Lea, Flood 2014), published test vector for seed 1234567
    L = O.lib()
    gamma = 0x9E3779B97F4A7C15
    s = 1234567
    assert L.oracle_splitmix64(s) == 6457827717110365317
    assert L.oracle_splitmix64((s + gamma) % 2**64) == 3203168211198807973


def test_generators_are_counter_based_and_plausible():
    a = O.fill("bytes", 1003, 2, 3)
    b = O.fill("bytes", 4096, 2, 3)
    assert np.array_equal(a[:1000], b[:1000])                # prefix property
    assert not np.array_equal(O.fill("bytes", 64, 2, 4), b[:64])   # PEs differ
    f = O.fill("f32", 1 << 18, 3, 0)
    assert abs(f.mean()) < 0.01 and abs(f.std() - 1) < 0.01
    hist = np.bincount(O.fill("bytes", 1 << 18, 2, 0), minlength=256)
    assert hist.min() > 800 and hist.max() < 1250


# ---------------------------------------------------------------------------------------------
# MoE routing / plan: brute force re-derivation on a small configuration
# ---------------------------------------------------------------------------------------------
def test_moe_routing_properties():
    npes, T, K, E = 4, 2000, 8, 64
    ex = O.moe_routing(npes, T, K, E, 1.1, 8).reshape(npes, T, K)
    assert ex.min() >= 0 and ex.max() < E
    assert all(len(set(row)) == K for row in ex[0])          # distinct experts per token
    freq = np.bincount(ex.ravel(), minlength=E)
    assert freq[0] > freq[7] > freq[40]                      # Zipf: low ranks dominate
    assert not np.array_equal(ex[0], ex[1])
    # first draw of every token follows the Zipf law closely: P(rank 1) = 1 / H_{E,1.1}
    p1 = 1.0 / sum(k ** -1.1 for k in range(1, E + 1))
    first = (ex[:, :, 0] == 0).mean()
    assert abs(first - p1) < 0.02


def test_moe_plan_brute_force():
    npes, T, K, E = 4, 50, 3, 16
    epp = E // npes
    ex = O.moe_routing(npes, T, K, E, 1.1, 8)
    counts, seg_base, dest_pe, dest_row, recv_rows = O.moe_plan(ex, npes, T, K, E)
    # receive buffer of PE d: rows sorted by (expert, source PE, (token, k) order)
    for d in range(npes):
        order = []
        for e in range(d * epp, (d + 1) * epp):
            for src in range(npes):
                for r in range(T * K):
                    if ex[src, r] == e:
                        order.append((src, r))
        assert recv_rows[d] == len(order)
        for row, (src, r) in enumerate(order):
            assert dest_pe[src, r] == d and dest_row[src, r] == row
    assert counts.sum() == npes * T * K
    for e in range(E):
        for src in range(npes):
            assert counts[src, e] == (ex[src] == e).sum()
    # dispatch then combine returns every token copy to its slot
    rng = np.random.default_rng(0)
    send = rng.integers(0, 256, (npes, T, 24), dtype=np.uint8)
    recv = O.moe_dispatch(send, dest_pe, dest_row, recv_rows, T, K)
    for src in range(npes):
        for r in range(T * K):
            assert np.array_equal(recv[dest_pe[src, r]][dest_row[src, r]], send[src, r // K])
    back = O.moe_combine(recv, dest_pe, dest_row, T, K, 24)
    assert np.array_equal(back, np.repeat(send, K, axis=1))


# ---------------------------------------------------------------------------------------------
# broadcast / reducescatter
# ---------------------------------------------------------------------------------------------
def test_broadcast_brute_force_and_reference_known_answer():
    rng = np.random.default_rng(4)
    for npes, nbytes, root in ((1, 5, 0), (3, 7, 2), (8, 64, 5)):
        src = rng.integers(0, 256, (npes, nbytes), dtype=np.uint8)
        got = O.broadcast(src, root)
        for q in range(npes):
            assert np.array_equal(got[q], src[root])
    # examples/ring-bcast.cu:44-72: the root (PE 0) holds mype + i = i, every PE ends with i
    npes, n = 4, 100
    data = np.stack([(pe + np.arange(n)).astype(np.int32) for pe in range(npes)])
    got = O.broadcast(data.view(np.uint8), 0).view(np.int32)
    assert all((got[pe] == np.arange(n)).all() for pe in range(npes))


def test_reducescatter_is_the_sliced_reduce_and_keeps_its_operand_order():
    rng = np.random.default_rng(6)
    npes, n = 5, 37
    # order-free operators: PE q's result is slice q of the (already pinned) allreduce
    for kind in ("i32", "u64", "i8"):
        dt = O.NP_STORAGE[kind]
        info = np.iinfo(dt)
        src = rng.integers(info.min, info.max, (npes, npes * n), dtype=dt, endpoint=True)
        for op in ("sum", "xor", "min", "prod"):
            got = O.reducescatter(kind, op, src)
            want = O.reduce(kind, op, src).reshape(npes, n)
            assert np.array_equal(got, want), (kind, op)
    # fp32 sum: numpy left fold acc = acc + x_p
    f = (rng.standard_normal((npes, npes * n)) * 10.0 ** rng.integers(-5, 6, (npes, npes * n))).astype(np.float32)
    acc = f[0].copy()
    for p in range(1, npes):
        acc = acc + f[p]
    assert np.array_equal(O.reducescatter("f32", "sum", f).reshape(-1), acc)

    # operand order acc = op(acc, x) with max(a, b) = (a > b) ? a : b, evaluated by hand; the last
    # case tells it apart from the allreduce order acc = op(x, acc), which gives NaN there
    def rs_max(xs):
        col = np.array(xs, np.float32)[:, None]
        return O.reducescatter("f32", "max", np.tile(col, (1, len(xs))))[0, 0]
    nan = float("nan")
    assert np.isnan(rs_max([1, 2, nan]))      # max(1,2)=2 ; (2>nan)?2:nan = nan
    assert rs_max([nan, 1, 2]) == 2.0         # (nan>1)?nan:1 = 1 ; (1>2)?1:2 = 2
    assert rs_max([1, nan, 0]) == 0.0         # (1>nan)?1:nan = nan ; (nan>0)?nan:0 = 0
    assert np.isnan(O.reduce("f32", "max", np.array([[1], [nan], [0]], np.float32))[0])


# ---------------------------------------------------------------------------------------------
# team arithmetic: PE sets enumerated from the definitions
# ---------------------------------------------------------------------------------------------
def test_team_split_strided_enumerates_the_parent_members_by_index():
    npes = 24
    parents = [(0, 1, 24), (0, 1, 8), (3, 2, 10), (1, 5, 4), (23, 1, 1)]
    for parent in parents:
        members = O.team_members(parent)             # parent index -> world PE
        for start in range(-1, parent[2] + 1):
            for stride in range(0, 5):
                for size in range(0, parent[2] + 2):
                    got = O.team_split_strided(parent, npes, start, stride, size)
                    ok = 0 <= start < parent[2] and 1 <= size <= parent[2] and stride >= 1
                    want = None
                    if ok:
                        idx = [start + i * stride for i in range(size)]
                        # the reference checks the world PEs, not the parent's bounds
                        world = [parent[0] + j * parent[1] for j in idx]
                        if world[0] < npes and world[-1] < npes:
                            want = world
                    if want is None:
                        assert got is None, (parent, start, stride, size)
                    else:
                        assert got is not None and O.team_members(got) == want, (parent, start, stride, size)
                        if idx[-1] < parent[2]:
                            assert want == [members[j] for j in idx]
    # the gemm_allreduce example duplicates the world team: examples/gemm_allreduce/...:434
    assert O.team_split_strided((0, 1, 8), 8, 0, 1, 8) == (0, 1, 8)


def test_team_translate_pe_against_set_lookup():
    teams = [(0, 1, 16), (0, 2, 8), (1, 2, 8), (4, 3, 4), (5, 1, 1), (0, 4, 4)]
    for src in teams:
        sm = O.team_members(src)
        for dst in teams:
            dm = O.team_members(dst)
            for i in range(src[2]):
                want = dm.index(sm[i]) if sm[i] in dm else -1
                assert O.team_translate_pe(src, i, dst) == want, (src, i, dst)
            # the reference wraps an index equal to the size to member 0 and rejects larger ones
            assert O.team_translate_pe(src, src[2], dst) == (dm.index(sm[0]) if sm[0] in dm else -1)
            assert O.team_translate_pe(src, src[2] + 1, dst) == -1
            assert O.team_translate_pe(src, -1, dst) == -1


def test_team_split_2d_rows_and_columns_partition_the_parent():
    for parent in [(0, 1, 16), (0, 1, 10), (2, 3, 7), (0, 1, 1), (1, 2, 12)]:
        members = O.team_members(parent)
        n = parent[2]
        for xrange_ in (1, 2, 3, 4, 5, n, n + 3):
            xr = min(xrange_, n)
            rows, cols = {}, {}
            for i in range(n):                       # row-major grid of parent indices
                rows.setdefault(i // xr, []).append(members[i])
                cols.setdefault(i % xr, []).append(members[i])
            for i in range(n):
                x, y = O.team_split_2d(parent, xrange_, i)
                assert O.team_members(x) == rows[i // xr], (parent, xrange_, i)
                assert O.team_members(y) == cols[i % xr], (parent, xrange_, i)


# ---------------------------------------------------------------------------------------------
# atomic memory operations against Python integers
# ---------------------------------------------------------------------------------------------
def _amo_python(op, bits, cur, val, cond):
    m = (1 << bits) - 1
    cur, val, cond = cur & m, val & m, cond & m
    new = {"inc": cur + 1, "fetch_inc": cur + 1, "set": val, "swap": val, "add": cur + val,
           "fetch_add": cur + val, "and": cur & val, "fetch_and": cur & val, "or": cur | val,
           "fetch_or": cur | val, "xor": cur ^ val, "fetch_xor": cur ^ val, "fetch": cur,
           "compare_swap": val if cur == cond else cur}[op]
    return new & m, cur


def test_amo_semantics_against_python_integers():
    rng = np.random.default_rng(21)
    edge = [0, 1, 2, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF, 0x100000000, 2**63 - 1, 2**63, 2**64 - 1]
    for bits in (32, 64):
        words = edge + [int(x) for x in rng.integers(0, 2**64, 40, dtype=np.uint64)]
        for op in O.AMO:
            for cur in words:
                for val in words[:12] + words[-6:]:
                    for cond in (cur, cur ^ 1, val):
                        assert O.amo(op, bits, cur, val, cond) == _amo_python(op, bits, cur, val, cond), \
                            (op, bits, cur, val, cond)
    # wrap-around and the compare_swap miss, by hand
    assert O.amo("fetch_add", 32, 0xFFFFFFFF, 2) == (1, 0xFFFFFFFF)
    assert O.amo("inc", 64, 2**64 - 1) == (0, 2**64 - 1)
    assert O.amo("compare_swap", 64, 5, 9, 4) == (5, 5) and O.amo("compare_swap", 64, 5, 9, 5) == (9, 5)


def test_maxloc_reduce_is_argmax_with_later_pe_winning_ties():
    # operator (a.x > b.x) ? a : b folded from PE 0 upwards (reduce.cuh:107-111, :1738-1747)
    rng = np.random.default_rng(21)
    npes, n = 7, 300
    vals = rng.standard_normal((npes, n))
    locs = rng.integers(0, 1 << 20, (npes, n)).astype(np.float64)
    got = O.maxloc_reduce(np.stack([vals, locs], axis=2))
    win = vals.argmax(axis=0)                                   # distinct values: plain argmax
    for q in range(npes):
        assert np.array_equal(got[q, :, 0], vals.max(axis=0))
        assert np.array_equal(got[q, :, 1], locs[win, np.arange(n)])
    # equal values: the pair of the LAST PE holding the maximum comes out
    tie = np.array([[[5.0, 10.0]], [[7.0, 11.0]], [[7.0, 12.0]], [[3.0, 13.0]]])
    assert np.array_equal(O.maxloc_reduce(tie)[0, 0], [7.0, 12.0])
    # signed zeros compare equal: the later one wins, with its sign
    z = np.array([[[0.0, 1.0]], [[-0.0, 2.0]]])
    out = O.maxloc_reduce(z)[1, 0]
    assert out[1] == 2.0 and np.signbit(out[0])
    # NaN: a NaN met as the new operand replaces the accumulator, and is dropped by the next one
    nan = float("nan")
    def fold(values):
        return O.maxloc_reduce(np.array([[[v, float(i)]] for i, v in enumerate(values)]))[0, 0]
    assert np.isnan(fold([1.0, 2.0, nan])[0]) and fold([1.0, 2.0, nan])[1] == 2.0
    assert np.array_equal(fold([nan, 1.0, 2.0]), [2.0, 2.0])
    assert np.array_equal(fold([1.0, nan, 0.0]), [0.0, 2.0])
    assert np.array_equal(fold([4.0]), [4.0, 0.0])              # a single PE: its own pair
