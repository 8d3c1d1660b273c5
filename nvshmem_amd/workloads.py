"""The measured workloads, defined once: bench.py times and verifies them, profile_workloads.py
runs the same objects under rocprofv3.

A Group owns one runtime's buffers (a symmetric heap of `heap_bytes` per PE, inputs uploaded once);
its Items are the timed calls.  An Item's step() enqueues ONE pass of the workload on the null stream
and returns nothing; `algorithmic_bytes` is what one step must move at least (each source byte read
once, each destination byte written once), the figure the HBM roofline is priced on.

Inputs come from a generator `gen(kind, npes, n, seed) -> [npes, n] array` (kinds: bytes, u64, i32, f32,
bf16 as uint16), so that the benchmark can use the oracle's seeded streams and the profiler plain numpy
noise; nothing here imports the oracle.
"""
import numpy as np

from . import _lib
from .host import SCOPE_BLOCK, SCOPE_WARP, TEAM_WORLD

MiB = 1 << 20
HEADLINE = "put_block_256MiB_16blk"


class Item:
    def __init__(self, name, dtype, algorithmic_bytes, kernel, workload, step, config=None, scale=1):
        self.name, self.dtype, self.algorithmic_bytes = name, dtype, algorithmic_bytes
        self.kernel, self.workload, self.step = kernel, workload, step
        self.config = dict(config or {})
        self.scale = scale          # divides the requested number of steps (very long steps)
        self.cache_resident = False  # True: the working set stays in the 256 MiB Infinity Cache between steps,
                                     # so its rate is not an HBM figure and no fraction of the HBM peak is quoted


class Group:
    kind = ""
    npes = 8
    heap_bytes = 0

    def names(self):
        """Names of the items setup() returns, without a GPU."""
        raise NotImplementedError

    def setup(self, rt, gen):
        raise NotImplementedError


def _check(rc, what, rt):
    if rc != 0:
        raise RuntimeError("%s failed: %d %s" % (what, rc, rt.last_error()))


# ------------------------------------------------------------------------------------------------
# put / get: PE p <-> (p + 1) % npes, the sweep's two largest sizes at 1 / 4 / 16 blocks of 1024
# threads per PE (block b moves the b-th contiguous slice), plus the launch shape that fills the GPU
# ------------------------------------------------------------------------------------------------
class RingRma(Group):
    kind = "rma"
    npes = 8
    SIZES = (64 * MiB, 256 * MiB)
    BLOCKS = (1, 4, 16)
    THREADS = 1024
    FILLED = (262144, 64)          # one wavefront per KiB

    def __init__(self):
        self.smax = max(self.SIZES)
        self.heap_bytes = 2 * self.smax + 64 * MiB

    def names(self):
        return ["%s_block_%dMiB_%dblk" % (w, s // MiB, b) for w in ("put", "get") for s in self.SIZES
                for b in self.BLOCKS] + ["put_block_256MiB_filled"]

    def setup(self, rt, gen):
        self.rt, self.perf = rt, rt.perftest()
        self.src = rt.malloc(self.smax)
        self.dst = rt.malloc(self.smax)
        self.data = gen("bytes", self.npes, self.smax, 2)
        rt.upload_all(self.src, self.data)
        rt.fill(self.dst, 0, self.smax)
        items = []
        for is_get in (0, 1):
            what = "get" if is_get else "put"
            for size in self.SIZES:
                for blocks in self.BLOCKS:
                    items.append(self._item("%s_block_%dMiB_%dblk" % (what, size // MiB, blocks), is_get, size,
                                            blocks, self.THREADS))
        items.append(self._item("put_block_256MiB_filled", 0, self.smax, *self.FILLED))
        return items

    def _item(self, name, is_get, size, blocks, threads):
        def step():
            _check(self.perf.nvshmem_perftest_ring_rma(self.dst, self.src, size, blocks, threads, SCOPE_BLOCK,
                                                       is_get, 1, None), name, self.rt)
        api = "nvshmemx_getmem_block" if is_get else "nvshmemx_putmem_block"
        return Item(name, "u8", 2 * self.npes * size,
                    "ring_rma_kernel<BLOCK, %s> (nvshmemi_memcpy_threadgroup)" % ("get" if is_get else "put"),
                    "%s: %s ring, %d logical PEs x %d MiB, %d blocks x %d threads per PE, block b moves the "
                    "b-th contiguous slice" % (name, api, self.npes, size // MiB, blocks, threads), step,
                    {"npes": self.npes, "bytes_per_pe": size, "blocks_per_pe": blocks, "threads_per_block": threads,
                     "is_get": is_get})


class StreamProbe(Group):
    """Counter probes, not API workloads (profile_workloads.py runs them, bench.py does not): the access
    pattern of the 16-block put with one side removed."""
    kind = "probe"
    npes = 8
    SIZE = 256 * MiB

    def __init__(self):
        self.heap_bytes = self.SIZE + 64 * MiB

    # (name, blocks per PE, threads, mode: 0 read, 1 write with streaming stores, 2 write with write-through stores)
    SHAPES = (("stream_read_16blk", 16, 1024, 0), ("stream_write_16blk", 16, 1024, 1), ("stream_write_8blk", 8, 1024, 1),
              ("stream_read_filled", 1024, 256, 0), ("stream_write_filled", 32768, 64, 1),
              ("stream_write_through_filled", 32768, 64, 2))

    def names(self):
        return [s[0] for s in self.SHAPES]

    def setup(self, rt, gen):
        perf = rt.perftest()
        buf = rt.malloc(self.SIZE)
        rt.upload_all(buf, gen("bytes", self.npes, self.SIZE, 2))
        items = []
        for name, blocks, threads, mode in self.SHAPES:
            def step(name=name, blocks=blocks, threads=threads, mode=mode):
                _check(perf.nvshmem_perftest_stream_probe(buf, self.SIZE, blocks, threads, mode, None), name, rt)
            what = ("read", "write with streaming (nt) stores", "write with write-through (sc1 nt) stores")[mode]
            items.append(Item(name, "u8", self.npes * self.SIZE, "stream_probe_kernel<%d>" % mode,
                              "%s: counter probe, not an API call - %d blocks x %d threads per PE %s their slice of 256 MiB "
                              "per PE in the access pattern of the long block-scoped copy, the other side removed"
                              % (name, blocks, threads, what), step,
                              {"npes": self.npes, "bytes_per_pe": self.SIZE, "blocks_per_pe": blocks,
                               "threads_per_block": threads}))
        return items


# ------------------------------------------------------------------------------------------------
# allreduce on a stream
# ------------------------------------------------------------------------------------------------
class Reduce(Group):
    kind = "reduce"
    # (name, API type, op, generator kind, numpy storage, element bytes, seed)
    def __init__(self, npes, n, variants, tag):
        self.npes, self.n, self.variants, self.tag = npes, n, variants, tag
        self.heap_bytes = 2 * n * 8 + 64 * MiB

    def names(self):
        return [v[0] for v in self.variants]

    def setup(self, rt, gen):
        self.rt = rt
        self.src = rt.malloc(self.n * 8)
        self.dst = rt.malloc(self.n * 8)
        self.gen = gen
        self.data = {}
        items = []
        for name, type_name, op, kind, es, seed in self.variants:
            fn = _lib.typed_coll(rt.lib, "nvshmemx_%s_%s_reduce_on_stream" % (type_name, op), True)

            def prepare(kind=kind, seed=seed):
                if self.data.get("kind") != (kind, seed):
                    d = self.gen(kind, self.npes, self.n, seed)
                    self.rt.upload_all(self.src, d)
                    self.data = {"kind": (kind, seed), "array": d}

            def step(fn=fn, name=name):
                _check(fn(TEAM_WORLD, self.dst, self.src, self.n, None), name, self.rt)
            it = Item(name, {"float": "f32", "bfloat16": "bf16", "int32": "i32", "int64": "i64"}[type_name],
                      2 * self.npes * self.n * es,
                      "reduce_vector_kernel / reduce_gather_kernel <%s, %s>" % (type_name, op),
                      "%s: nvshmemx_%s_%s_reduce_on_stream, %d logical PEs x %d elements (%s), fixed PE order"
                      % (name, type_name, op, self.npes, self.n, self.tag), step,
                      {"npes": self.npes, "nreduce": self.n, "type": type_name, "op": op})
            it.prepare, it.oracle_dtype, it.op, it.elem_bytes = prepare, kind, op, es
            it.cache_resident = 2 * self.npes * self.n * es <= 256 * MiB
            items.append(it)
        return items


CONFIG1 = (("sum_reduce_int32_1Mi", "int32", "sum", "i32", 4, 1),)
CONFIG3 = (("sum_reduce", "float", "sum", "f32", 4, 3), ("max_reduce_fp32", "float", "max", "f32", 4, 3),
           ("sum_reduce_bf16", "bfloat16", "sum", "bf16", 2, 4), ("max_reduce_bf16", "bfloat16", "max", "bf16", 2, 4),
           ("xor_reduce_int64", "int64", "xor", "u64", 8, 5))


# ------------------------------------------------------------------------------------------------
# fcollect + alltoall (config 4: 16 PEs x 2^22 elements, fp32 and int64), and a 1 GiB alltoall whose
# source cannot stay in the Infinity Cache
# ------------------------------------------------------------------------------------------------
class Collect(Group):
    kind = "collect"
    npes = 16

    def __init__(self, type_name, es, n, with_fcollect=True, suffix=""):
        self.type_name, self.es, self.n, self.with_fcollect, self.suffix = type_name, es, n, with_fcollect, suffix
        self.heap_bytes = (2 + (self.npes if with_fcollect else 0)) * n * es + 16 * MiB

    def names(self):
        label = {"float": "fp32", "int64": "int64"}[self.type_name]
        return ["alltoall_%s%s" % (label, self.suffix)] + (["fcollect_%s" % label] if self.with_fcollect else [])

    def setup(self, rt, gen):
        self.rt = rt
        n, es, npes = self.n, self.es, self.npes
        self.src = rt.malloc(n * es)
        self.a2a_dst = rt.malloc(n * es)
        self.data = gen("u64", npes, n * es // 8, 6).view(np.uint8).reshape(npes, -1)
        rt.upload_all(self.src, self.data)
        a2a = _lib.typed_coll(rt.lib, "nvshmemx_%s_alltoall_on_stream" % self.type_name, True)
        cached = npes * n * es <= 256 * MiB

        def a2a_step():
            _check(a2a(TEAM_WORLD, self.a2a_dst, self.src, n // npes, None), "alltoall", rt)
        label = {"float": "fp32", "int64": "int64"}[self.type_name]
        items = [Item("alltoall_%s%s" % (label, self.suffix), "u8", 2 * npes * n * es, "segment_copy_kernel<alltoall>",
                      "alltoall: nvshmemx_%s_alltoall_on_stream, %d logical PEs x %d elements, block %d elements per "
                      "destination" % (self.type_name, npes, n, n // npes), a2a_step,
                      {"npes": npes, "nelems": n // npes, "type": self.type_name,
                       "note": ("the %d MiB of sources fit the Infinity Cache and are re-read from it on repeated steps: "
                                "not an HBM-bound figure" % (npes * n * es // MiB) if cached else
                                "sources larger than the Infinity Cache: HBM-bound")})]
        items[0].what = "alltoall"
        items[0].cache_resident = cached
        if self.with_fcollect:
            self.fc_dst = rt.malloc(npes * n * es)
            fc = _lib.typed_coll(rt.lib, "nvshmemx_%s_fcollect_on_stream" % self.type_name, True)

            def fc_step():
                _check(fc(TEAM_WORLD, self.fc_dst, self.src, n, None), "fcollect", rt)
            it = Item("fcollect_%s" % label, "u8", (npes + 1) * npes * n * es, "segment_copy_kernel<fcollect>",
                      "fcollect: nvshmemx_%s_fcollect_on_stream, %d logical PEs x %d elements" % (self.type_name, npes, n),
                      fc_step, {"npes": npes, "nelems": n, "type": self.type_name})
            it.what = "fcollect"
            items.append(it)
        return items


class Reducescatter(Group):
    kind = "reducescatter"
    npes = 8

    def __init__(self, n=1 << 23):
        self.n = n
        self.heap_bytes = 9 * n * 4 + 64 * MiB

    def names(self):
        return ["reducescatter"]

    def setup(self, rt, gen):
        self.rt = rt
        n, npes = self.n, self.npes
        self.src = rt.malloc(npes * n * 4)
        self.dst = rt.malloc(n * 4)
        self.data = gen("f32", npes, npes * n, 9)
        rt.upload_all(self.src, self.data)
        fn = _lib.typed_coll(rt.lib, "nvshmemx_float_sum_reducescatter_on_stream", True)

        def step():
            _check(fn(TEAM_WORLD, self.dst, self.src, n, None), "reducescatter", rt)
        return [Item("reducescatter", "f32", (npes + 1) * npes * n * 4, "reducescatter_gather_kernel<float, sum, 8>",
                     "reducescatter: nvshmemx_float_sum_reducescatter_on_stream, 8 logical PEs, source 8 x 2^23 fp32 "
                     "(256 MiB) per PE, result 2^23 fp32 per PE", step, {"npes": npes, "nreduce": n})]


class Broadcast(Group):
    kind = "broadcast"
    npes = 8

    def __init__(self, nbytes=512 * MiB, root=3):
        self.nbytes, self.root = nbytes, root
        self.heap_bytes = 2 * nbytes + 64 * MiB

    def names(self):
        return ["broadcast"]

    def setup(self, rt, gen):
        self.rt = rt
        self.src = rt.malloc(self.nbytes)
        self.dst = rt.malloc(self.nbytes)
        self.row = gen("bytes", 1, self.nbytes, 12)[0]
        rt.upload(self.src, self.root, self.row)

        def step():
            _check(rt.lib.nvshmemx_broadcastmem_on_stream(TEAM_WORLD, self.dst, self.src, self.nbytes, self.root, None),
                   "broadcast", rt)
        return [Item("broadcast", "u8", (self.npes + 1) * self.nbytes, "segment_copy_kernel<broadcast>",
                     "broadcast: nvshmemx_broadcastmem_on_stream, 8 logical PEs, %d MiB from PE %d (larger than the "
                     "Infinity Cache)" % (self.nbytes // MiB, self.root), step,
                     {"npes": self.npes, "bytes": self.nbytes, "root": self.root})]


# ------------------------------------------------------------------------------------------------
# MoE token shuffle (config 5)
# ------------------------------------------------------------------------------------------------
class MoeShuffle(Group):
    kind = "moe"
    npes, T, K, E, row = 8, 8192, 8, 256, 7168 * 2
    SIG_STRIDE = 16     # one 128-byte line per signal word

    def __init__(self, plan):
        """plan = (dest_pe, dest_row [npes, T*K], expected [dst, src] uint64, recv_rows [npes])."""
        self.dest_pe, self.dest_row, self.expected, self.recv_rows = plan
        self.cap = int(self.recv_rows.max())
        self.rows = self.T * self.K
        self.heap_bytes = self.cap * self.row + self.rows * self.row + self.T * self.row + 64 * MiB

    FULL_ORDER_TOKENS = 512     # the reference-order row runs on the first tokens of every PE only: it takes 16x as long per row

    def names(self):
        return ["moe_dispatch_put_signal", "moe_dispatch_put_signal_full_order", "moe_dispatch_put_quiet_signal",
                "moe_dispatch_plain_store", "moe_combine"]

    def setup(self, rt, gen):
        self.rt, self.perf = rt, rt.perftest()
        npes, T, K, row, cap, rows = self.npes, self.T, self.K, self.row, self.cap, self.rows
        self.send = rt.malloc(T * row); self.recv = rt.malloc(cap * row); self.out = rt.malloc(rows * row)
        self.d_pe = rt.malloc(rows * 4); self.d_row = rt.malloc(rows * 8)
        self.d_expected = rt.malloc(npes * 8)
        self.sig = rt.calloc(npes * self.SIG_STRIDE, 8)
        rt.upload_all(self.d_pe, self.dest_pe); rt.upload_all(self.d_row, self.dest_row)
        rt.upload_all(self.d_expected, self.expected)
        # the rows of the first FULL_ORDER_TOKENS tokens of every PE, counted per (destination, source)
        Ts = self.FULL_ORDER_TOKENS
        head = self.dest_pe[:, :Ts * K]
        self.expected_head = np.stack([[int((head[s] == d).sum()) for s in range(npes)]
                                       for d in range(npes)]).astype(np.uint64)
        self.d_expected_head = rt.malloc(npes * 8)
        rt.upload_all(self.d_expected_head, self.expected_head)
        self.payload = gen("u64", npes, T * row // 8, 7).view(np.uint8).reshape(npes, T, row)
        rt.upload_all(self.send, self.payload)
        perf = self.perf

        def put_signal():
            # plain NVSHMEM_SIGNAL_ADD at the call sites; the payload-only order comes from the library option
            # that NVSHMEM_AMD_PUT_SIGNAL_ORDER=payload sets, as for a program written for the reference
            # (set by the item's prepare(), outside the timed steps)
            _check(perf.nvshmem_perftest_fill_words(self.sig, 0, npes * self.SIG_STRIDE, None), "fill_words", rt)
            _check(perf.nvshmem_perftest_moe_dispatch_put_signal(
                self.recv, cap, self.send, self.d_pe, self.d_row, self.d_expected, self.sig, self.SIG_STRIDE, T, K,
                row, 64, 256, SCOPE_WARP | 256, None), "moe_dispatch_put_signal", rt)

        def put_signal_full_order():
            _check(perf.nvshmem_perftest_fill_words(self.sig, 0, npes * self.SIG_STRIDE, None), "fill_words", rt)
            _check(perf.nvshmem_perftest_moe_dispatch_put_signal(
                self.recv, cap, self.send, self.d_pe, self.d_row, self.d_expected_head, self.sig, self.SIG_STRIDE,
                self.FULL_ORDER_TOKENS, K, row, 64, 256, SCOPE_WARP | 256, None), "moe_dispatch_put_signal", rt)

        def put_quiet_signal():
            _check(perf.nvshmem_perftest_fill_words(self.sig, 0, npes, None), "fill_words", rt)
            _check(perf.nvshmem_perftest_moe_dispatch_ex(self.recv, cap, self.send, self.d_pe, self.d_row,
                                                         self.d_expected, self.sig, T, K, row, 32, 256, SCOPE_WARP,
                                                         None), "moe_dispatch_ex", rt)

        def plain_store():
            _check(perf.nvshmem_perftest_fill_words(self.sig, 0, npes, None), "fill_words", rt)
            _check(perf.nvshmem_perftest_moe_dispatch_pieces(self.recv, cap, self.send, self.d_pe, self.d_row,
                                                             self.d_expected, self.sig, T, K, row, 1024, 256, None),
                   "moe_dispatch_pieces", rt)

        def combine():
            # one block (one wavefront) per 2 KiB work item: 7 items per 14 KiB row
            _check(perf.nvshmem_perftest_moe_combine_pieces(self.out, self.recv, cap, self.d_pe, self.d_row, T, K, row,
                                                            2048, rows * ((row + 2047) // 2048), 64, SCOPE_WARP, None),
                   "moe_combine", rt)
        moved = npes * rows * row
        shape = "8 logical PEs x 8192 tokens x 7168 bf16, top-8 of 256 experts, Zipf(1.1)"
        common = {"npes": npes, "tokens": T, "topk": K, "experts": self.E, "row_bytes": row}
        lower = ("algorithmic bytes = every source row read once and written top-k times (7.875 GiB); the timed "
                 "step includes clearing the signal words")
        items = [
            Item("moe_dispatch_put_signal", "u8", moved + moved // K,
                 "moe_dispatch_rowsignal_kernel<warp> (nvshmemx_putmem_signal_nbi_warp per row)",
                 "moe_dispatch_put_signal: one nvshmemx_putmem_signal_nbi_warp per row copy (plain NVSHMEM_SIGNAL_ADD of 1 "
                 "at the call sites, payload-only order chosen library-wide as NVSHMEM_AMD_PUT_SIGNAL_ORDER=payload "
                 "does, one signal word per source on its own 128-byte line), receivers "
                 "nvshmem_signal_wait_until(GE); " + shape, put_signal, dict(common, note=lower), scale=5),
            Item("moe_dispatch_put_signal_full_order", "u8", (moved + moved // K) * self.FULL_ORDER_TOKENS // T,
                 "moe_dispatch_rowsignal_kernel<warp> (nvshmemx_putmem_signal_nbi_warp per row, reference order)",
                 "moe_dispatch_put_signal_full_order: the same kernel with the library's default order of the signal, "
                 "the reference's (a full release in front of every signal: an L2 write-back per row), on the first "
                 "%d tokens of every PE; " % self.FULL_ORDER_TOKENS + shape, put_signal_full_order,
                 dict(common, tokens=self.FULL_ORDER_TOKENS,
                      note="a cost on record, not a rate to compare: what an unmodified caller pays per row until it "
                           "opts into the payload-only order"), scale=5),
            Item("moe_dispatch_put_quiet_signal", "u8", moved + moved // K,
                 "moe_dispatch_kernel<warp> (nvshmemx_putmem_nbi_warp per row, nvshmemx_quiet_block, nvshmemx_signal_op)",
                 "moe_dispatch_put_quiet_signal: one nvshmemx_putmem_nbi_warp per row copy, rows per destination "
                 "tallied per block, then one nvshmemx_quiet_block and one nvshmemx_signal_op(NVSHMEM_SIGNAL_ADD) per "
                 "block and destination, receivers nvshmem_signal_wait_until(GE); " + shape, put_quiet_signal,
                 dict(common, note=lower), scale=5),
            Item("moe_dispatch_plain_store", "u8", moved + moved // K,
                 "moe_dispatch_direct_kernel<1> + moe_dispatch_signal_kernel",
                 "moe_dispatch_plain_store: NOT the put API - 1 KiB work items stored through nvshmem_ptr by one "
                 "kernel, then a second kernel adds the row counts to the signal words and waits "
                 "(signal_wait_until GE); the kernel boundary orders rows before signals; " + shape, plain_store,
                 dict(common, note=lower), scale=5),
            Item("moe_combine", "u8", 2 * moved, "moe_combine_kernel<warp, 2048>",
                 "moe_combine: nvshmemx_getmem_nbi_warp per 2 KiB of a row; " + shape, combine, common, scale=5),
        ]
        for it, what in zip(items, ("put_signal", "put_signal_head", "plain_store", "plain_store", "combine")):
            it.what = what
            # the library-wide order of put-with-signal: payload-only for the first row, the default for the rest
            it.prepare = (lambda on=(what == "put_signal"): rt.lib.nvshmemx_amd_set_put_signal_order(1 if on else 0))

        def prepare_combine():
            # the combine gathers what a dispatch delivered: run one (whatever ran before may have sent a part only)
            rt.lib.nvshmemx_amd_set_put_signal_order(0)
            plain_store()
        items[-1].prepare = prepare_combine
        return items


def team_size_variant(npes):
    return (("sum_reduce_fp32_%dpe" % npes, "float", "sum", "f32", 4, 3),)


def profile_only_groups():
    """Groups that only the profiler runs (counter probes)."""
    return [StreamProbe()]


def all_groups(moe_plan):
    """The groups in the order bench.py reports them.  moe_plan: see MoeShuffle."""
    return [RingRma(),
            Reduce(8, 1 << 20, CONFIG1, "config 1"),
            Reduce(8, 1 << 26, CONFIG3, "config 3: 256 MiB of fp32 per PE"),
            # the same allreduce at other team sizes, 1 to 2 GiB of sources in all
            Reduce(4, 1 << 26, team_size_variant(4), "4 members x 256 MiB"),
            Reduce(16, 1 << 25, team_size_variant(16), "16 members x 128 MiB"),
            Reduce(64, 1 << 23, team_size_variant(64), "64 members x 32 MiB"),
            Collect("float", 4, 1 << 22),
            Collect("int64", 8, 1 << 22),
            Collect("float", 4, 1 << 24, with_fcollect=False, suffix="_1GiB"),
            Reducescatter(),
            Broadcast(),
            MoeShuffle(moe_plan)]
