"""GPU parity of the exported primitives against the CPU oracle (bit-exact), through the C ABI.

Shaped after the reference's own API tests
(test/ut/framework/communicator/impl/independent_op/data_api/ut_aicpu_ts_HcommLocalReduceOnThread.cc,
ut_aicpu_ts_HcommLocalCopyOnThread.cc) with real data instead of a mocked engine.
"""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, UNIT, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

# counts chosen to hit: empty, sub-vector, exact vector, one tile +- 1 element, several tiles + tail
COUNTS = [0, 1, 7, 16, 4099, 16384, 16385, 1 << 20, (1 << 20) + 13]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("nbytes", [0, 1, 15, 16, 17, 16384, 16400, 3 * 16384 + 5, (1 << 22) + 3])
def test_local_copy(gpu_thread, nbytes):
    say("copy", nbytes)
    src = np.random.default_rng(nbytes).integers(0, 256, nbytes + 64, dtype=np.uint8)
    d_src, d_dst = to_dev(src), to_dev(np.full(nbytes + 64, 0xAB, np.uint8))
    assert h.HcommLocalCopyOnThread(gpu_thread, d_dst.data_ptr(), d_src.data_ptr(), nbytes) == 0
    assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
    got = d_dst.cpu().numpy()
    assert np.array_equal(got[:nbytes], src[:nbytes])
    assert (got[nbytes:] == 0xAB).all(), "copy wrote past len"


@pytest.mark.parametrize("dst_off,src_off", [(1, 1), (3, 8), (16, 5), (2, 0)])
def test_local_copy_unaligned(gpu_thread, dst_off, src_off):
    nbytes = 100003
    say("copy unaligned", dst_off, src_off)
    src = np.random.default_rng(7).integers(0, 256, nbytes + 64, dtype=np.uint8)
    d_src, d_dst = to_dev(src), to_dev(np.full(nbytes + 64, 0xCD, np.uint8))
    assert h.HcommLocalCopyOnThread(gpu_thread, d_dst.data_ptr() + dst_off, d_src.data_ptr() + src_off, nbytes) == 0
    assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
    got = d_dst.cpu().numpy()
    assert np.array_equal(got[dst_off:dst_off + nbytes], src[src_off:src_off + nbytes])
    assert (got[:dst_off] == 0xCD).all() and (got[dst_off + nbytes:] == 0xCD).all()


def test_local_copy_same_pointer_is_noop(gpu_thread):
    d = to_dev(np.arange(64, dtype=np.uint8))
    h.HcommGfxLaunchLogClear(gpu_thread)
    assert h.HcommLocalCopyOnThread(gpu_thread, d.data_ptr(), d.data_ptr(), 64) == 0
    assert len(h.launch_log(gpu_thread)) == 0


@pytest.mark.parametrize("dtype", ["int8", "int16", "int32", "fp16", "fp32", "bf16"])
@pytest.mark.parametrize("op", ["sum", "max", "min"])
def test_local_reduce(gpu_thread, dtype, op):
    dt, o = DT[dtype], OPS[op]
    for count in COUNTS:
        for kind in ("default", "wide"):
            say("reduce", dtype, op, count, kind)
            a, b = gen(dt, count + 8, 11 + count, kind), gen(dt, count + 8, 29 + count, kind)
            want = a.copy()
            oracle.reduce(want[:count], b[:count].copy(), dt, o)
            d_a, d_b = to_dev(a), to_dev(b)
            assert h.HcommLocalReduceOnThread(gpu_thread, d_a.data_ptr(), d_b.data_ptr(), count, dt, o) == 0
            assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
            got = from_dev(d_a, a)
            assert_same(got[:count], want[:count], dt, "%s %s %d %s" % (dtype, op, count, kind))
            assert np.array_equal(got[count:], a[count:]), "reduce wrote past count"
            assert np.array_equal(from_dev(d_b, b), b), "reduce modified src"


@pytest.mark.parametrize("dtype", ["int8", "int32", "fp16", "fp32", "bf16"])
def test_local_reduce_prod_needs_opt_in(gpu_thread, dtype):
    """PROD is rejected by the primitive exactly as the reference does (cpu_primitives_c_adpt.cc:37)."""
    d = to_dev(np.zeros(64, np.uint8))
    assert h.HcommLocalReduceOnThread(gpu_thread, d.data_ptr(), d.data_ptr(), 4, DT[dtype], OPS["prod"]) == \
        h.HcclResult.E_PARA


@pytest.mark.parametrize("dtype", ["int8", "int16", "fp16", "fp32", "bf16"])
@pytest.mark.parametrize("op", ["sum", "max"])
@pytest.mark.parametrize("dst_el,src_el", [(1, 1), (1, 0), (3, 2)])
def test_local_reduce_unaligned(gpu_thread, dtype, op, dst_el, src_el):
    """Pointers offset by whole elements but not by 16 bytes take the element-wise kernel (only for the bytes up to
    the next 16-byte boundary when both operands are equally far from one)."""
    dt, o, count = DT[dtype], OPS[op], 70001
    say("reduce unaligned", dtype, op, dst_el, src_el)
    a, b = gen(dt, count + 16, 3), gen(dt, count + 16, 4)
    want = a.copy()
    oracle.reduce(want[dst_el:dst_el + count], b[src_el:src_el + count].copy(), dt, o)
    d_a, d_b = to_dev(a), to_dev(b)
    u = UNIT[dt]
    h.HcommGfxLaunchLogClear(gpu_thread)
    assert h.HcommLocalReduceOnThread(gpu_thread, d_a.data_ptr() + dst_el * u, d_b.data_ptr() + src_el * u, count,
                                      dt, o) == 0
    assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
    if dst_el == src_el and count * u >= 65536:  # equally misaligned and large: element-wise head, full-width body
        assert [r.kind for r in h.launch_log(gpu_thread)] == [h.Kernel.BYTEWISE, h.Kernel.REDUCE2]
    else:
        assert [r.kind for r in h.launch_log(gpu_thread)] == [h.Kernel.BYTEWISE]
    assert_same(from_dev(d_a, a), want, dt)


@pytest.mark.parametrize("dtype", ["int8", "bf16", "int32"])
def test_unaligned_operands_every_skew_and_length(gpu_thread, dtype):
    """The kernel for operands off 16-byte boundaries reads src in aligned vectors and puts every item together from
    its own and the next lane's: every distance of src from a 16-byte boundary (in whole elements) against several of
    dst's, for lengths of 0, 1, 2 items, one on either side of a wavefront's 64, of a workgroup's 256 and of a tile's
    1,024, and a few tiles with a ragged end; copy and reduce in ONE batch each (all segments of a skew in one
    launch), guard bytes before and behind every destination."""
    dt = DT[dtype]
    u = UNIT[dt]
    items = [0, 1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4099]
    rng = np.random.default_rng(77)
    for dst_skew in sorted({0, u, 16 - u, 8}):
        for src_skew in range(0, 16, u):
            say("unaligned skews", dtype, dst_skew, src_skew)
            cases = []
            for n_items in items:
                for extra in (0, u, 16 - u):        # bytes beyond the last whole item
                    nbytes = n_items * 16 + extra + ((16 - dst_skew) % 16 if n_items else 0)
                    if nbytes == 0:
                        continue
                    count = nbytes // u
                    a, b = gen(dt, count + 64 // u, int(rng.integers(1 << 30))), gen(dt, count + 64 // u, int(rng.integers(1 << 30)))
                    cases.append((count, a, b, to_dev(a), to_dev(b), to_dev(a)))
            for reduce in (False, True):
                assert h.HcommBatchModeStart(b"skews") == 0
                for count, a, b, d_a, d_b, d_c in cases:
                    dst = (d_a if reduce else d_c).data_ptr() + 16 + dst_skew
                    src = d_b.data_ptr() + 16 + src_skew
                    if reduce:
                        assert h.HcommLocalReduceOnThread(gpu_thread, dst, src, count, dt, oracle.SUM) == 0
                    else:
                        assert h.HcommLocalCopyOnThread(gpu_thread, dst, src, count * u) == 0
                assert h.HcommBatchModeEnd(b"skews") == 0
                assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
                for count, a, b, d_a, d_b, d_c in cases:
                    lo, so = (16 + dst_skew) // u, (16 + src_skew) // u
                    want = a.copy()
                    if reduce:
                        with np.errstate(all="ignore"):
                            oracle.reduce(want[lo:lo + count], b[so:so + count].copy(), dt, oracle.SUM)
                    else:
                        want[lo:lo + count] = b[so:so + count]
                    got = from_dev(d_a if reduce else d_c, a)
                    assert_same(got, want, dt, "%s skew %d/%d count %d %s" % (dtype, dst_skew, src_skew, count, "reduce" if reduce else "copy"))
                    assert np.array_equal(from_dev(d_b, b).view(np.uint8), b.view(np.uint8)), "src modified"


@pytest.mark.parametrize("shape", ["rows_few", "rows_many", "ragged", "unaligned"])
@pytest.mark.parametrize("reduce", [False, True])
def test_a_launch_gives_the_same_bytes_in_either_direction(gpu_thread, shape, reduce):
    """A large launch that reads what the launch before it wrote walks its table the other way (it starts on the bytes
    the memory-side cache still holds).  With the size from which that applies lowered to one byte, a chain of four
    dependent launches - dst (op)= src four times, or a copy passed on from buffer to buffer - runs forwards, backwards,
    forwards, backwards: same bytes as the oracle's, for the row grids with the short and the full argument table,
    the one-dimensional kernels (segments of very different lengths) and the kernel for unaligned operands, with
    element tails and guard bytes."""
    dt = DT["bf16"]
    u = UNIT[dt]
    counts = {"rows_few": [70001] * 5 + [69999], "rows_many": [33001 + (i % 3) for i in range(20)],
              "ragged": [5, 300007, 17, 65536, 1000001, 1], "unaligned": [70001, 8191, 300007]}[shape]
    skew = 1 if shape == "unaligned" else 0
    say("both directions", shape, reduce)
    rng = np.random.default_rng(5)
    lo, so, lo_c = 16 // u + skew, 16 // u + 3 * skew, 16 // u + 2 * skew   # no two of them equally far from a 16-byte boundary
    bufs = [(gen(dt, c + 32, int(rng.integers(1 << 30))), gen(dt, c + 32, int(rng.integers(1 << 30)))) for c in counts]
    dev = [(to_dev(a), to_dev(b), to_dev(a)) for a, b in bufs]   # dst, src, a second destination for the copy chain
    before = h.HcommGfxSetAlternateBytes(1)
    row_grids = h.HcommGfxSetDirectLaunches(1)   # as the caller has set it: this module also runs with them off
    h.HcommGfxSetDirectLaunches(row_grids)
    try:
        for hop in range(4):
            h.HcommGfxLaunchLogClear(gpu_thread)
            assert h.HcommBatchModeStart(b"dir") == 0
            for c, (d_a, d_b, d_c) in zip(counts, dev):
                if reduce:
                    assert h.HcommLocalReduceOnThread(gpu_thread, d_a.data_ptr() + lo * u, d_b.data_ptr() + so * u, c, dt,
                                                      oracle.SUM) == 0
                else:   # src -> a -> c -> a -> c, every hop reading what the hop before wrote
                    chain = [(d_b, so), (d_a, lo), (d_c, lo_c), (d_a, lo), (d_c, lo_c)]
                    (src, s_off), (dst, d_off) = chain[hop], chain[hop + 1]
                    assert h.HcommLocalCopyOnThread(gpu_thread, dst.data_ptr() + d_off * u, src.data_ptr() + s_off * u,
                                                    c * u) == 0
            assert h.HcommBatchModeEnd(b"dir") == 0
            log = h.launch_log(gpu_thread)
            assert len(log) == 1
            want_kind = h.Kernel.BYTEWISE if skew else (h.Kernel.REDUCE2 if reduce else h.Kernel.COPY)
            assert log[0].kind == want_kind and bool(log[0].rows) == (row_grids and shape.startswith("rows"))
            if hop == 0:   # forwards, unless the allocator handed out memory a launch of an earlier test wrote to
                first = log[0].backwards
            assert log[0].backwards == (first + hop) % 2
        assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
    finally:
        assert h.HcommGfxSetAlternateBytes(before) == 1
    for c, (a, b), (d_a, d_b, d_c) in zip(counts, bufs, dev):
        want = a.copy()
        if reduce:
            with np.errstate(all="ignore"):
                for hop in range(4):
                    oracle.reduce(want[lo:lo + c], b[so:so + c].copy(), dt, oracle.SUM)
            assert_same(from_dev(d_a, a), want, dt, "%s count %d" % (shape, c))
        else:
            want[lo:lo + c] = b[so:so + c]
            assert_same(from_dev(d_a, a), want, dt, "%s count %d, first destination" % (shape, c))
            want = a.copy()
            want[lo_c:lo_c + c] = b[so:so + c]
            assert_same(from_dev(d_c, a), want, dt, "%s count %d, second destination" % (shape, c))


def test_local_reduce_dst_equals_src(gpu_thread):
    """The reference's UT passes the same pointer for both operands; the result is x (op) x."""
    a = gen(oracle.F32, 5000, 5)
    d = to_dev(a)
    assert h.HcommLocalReduceOnThread(gpu_thread, d.data_ptr(), d.data_ptr(), 5000, oracle.F32, oracle.SUM) == 0
    h.HcommGfxThreadSynchronize(gpu_thread)
    assert_same(from_dev(d, a), a + a, oracle.F32)


SPECIAL_F32 = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.17549435e-38, 3.4028235e38,
                        -3.4028235e38, 65504.0, 65520.0, 2.0 ** -24, 2.0 ** -25, 1.0009765625, 0.333333343],
                       dtype=np.float32)


@pytest.mark.parametrize("dtype", ["fp16", "fp32", "bf16"])
@pytest.mark.parametrize("op", ["sum", "max", "min"])
def test_local_reduce_special_values(gpu_thread, dtype, op):
    """All pairs of special values: signed zeros, infinities, NaN, denormals, overflow to inf.
    MAX / MIN keep dst on ties and unordered comparisons; SUM of 16-bit types stores a canonical NaN."""
    dt, o = DT[dtype], OPS[op]
    if dt == oracle.F32:
        vals = SPECIAL_F32
    elif dt == oracle.F16:
        with np.errstate(over="ignore"):
            vals = SPECIAL_F32.astype(np.float16).view(np.uint16)
        vals = np.concatenate([vals, np.array([0x0001, 0x8001, 0x03FF, 0x7BFF, 0xFBFF, 0x7E01, 0xFE00], np.uint16)])
    else:
        vals = np.concatenate([(SPECIAL_F32.view(np.uint32) >> 16).astype(np.uint16),
                               np.array([0x0001, 0x8001, 0x007F, 0x7F7F, 0xFF7F, 0x7FC1, 0xFFC0], np.uint16)])
    a = np.repeat(vals, vals.size).copy()
    b = np.tile(vals, vals.size).copy()
    want = a.copy()
    with np.errstate(all="ignore"):
        oracle.reduce(want, b.copy(), dt, o)
    d_a, d_b = to_dev(a), to_dev(b)
    assert h.HcommLocalReduceOnThread(gpu_thread, d_a.data_ptr(), d_b.data_ptr(), a.size, dt, o) == 0
    h.HcommGfxThreadSynchronize(gpu_thread)
    assert_same(from_dev(d_a, a), want, dt, "%s %s specials" % (dtype, op))


def test_fp16_sum_exhaustive_against_oracle(gpu_thread):
    """Every fp16 bit pattern added to 512 partners (33.5 M pairs): conversions and rounding agree everywhere."""
    allh = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    partners = np.random.default_rng(3).integers(0, 1 << 16, 512, dtype=np.uint32).astype(np.uint16)
    a = np.tile(allh, partners.size)
    b = np.repeat(partners, allh.size)
    for dt in (oracle.F16, oracle.BF16):
        for o in (oracle.SUM, oracle.PROD):
            say("exhaustive", dt, o)
            if dt == oracle.BF16 and o == oracle.PROD:   # refused like the reference's collectives (param_check.cc:327-343)
                d = to_dev(np.zeros(64, np.uint8))
                assert h.HcommGfxReduceKOnThread(gpu_thread, d.data_ptr(), [d.data_ptr(), d.data_ptr()], 4, dt, o) == \
                    h.HcclResult.E_PARA
                continue
            want = a.copy()
            with np.errstate(all="ignore"):
                oracle.reduce(want, b.copy(), dt, o)
            d_a, d_b, d_o = to_dev(a), to_dev(b), to_dev(np.zeros_like(a))
            assert h.HcommGfxReduceKOnThread(gpu_thread, d_o.data_ptr(), [d_a.data_ptr(), d_b.data_ptr()], a.size, dt,
                                             o) == 0
            h.HcommGfxThreadSynchronize(gpu_thread)
            assert_same(from_dev(d_o, a), want, dt, "dt %d op %d" % (dt, o))


def test_batch_mode_merges_independent_ops(gpu_thread):
    """Eight reduces on disjoint buffers between Start and End become ONE launch; a dependent op splits."""
    dt, count = oracle.F32, 50000
    bufs = [gen(dt, count, 100 + i) for i in range(16)]
    dev = [to_dev(x) for x in bufs]
    h.HcommGfxThreadSynchronize(gpu_thread)
    h.HcommGfxLaunchLogClear(gpu_thread)
    assert h.HcommBatchModeStart(b"step") == 0
    for i in range(8):
        assert h.HcommLocalReduceOnThread(gpu_thread, dev[i].data_ptr(), dev[8 + i].data_ptr(), count, dt,
                                          oracle.SUM) == 0
    # depends on the first group's result: must not share its launch
    assert h.HcommLocalReduceOnThread(gpu_thread, dev[15].data_ptr(), dev[0].data_ptr(), count, dt, oracle.SUM) == 0
    assert len(h.launch_log(gpu_thread)) == 0, "batch mode must not launch before End"
    assert h.HcommBatchModeEnd(b"step") == 0
    h.HcommGfxThreadSynchronize(gpu_thread)
    log = h.launch_log(gpu_thread)
    assert [(r.kind, r.nseg) for r in log] == [(h.Kernel.REDUCE2, 8), (h.Kernel.REDUCE2, 1)]
    want = [x.copy() for x in bufs]
    for i in range(8):
        oracle.reduce(want[i], want[8 + i], dt, oracle.SUM)
    oracle.reduce(want[15], want[0], dt, oracle.SUM)
    for i in range(16):
        assert_same(from_dev(dev[i], bufs[i]), want[i], dt, "buf %d" % i)


@pytest.mark.parametrize("dtype,op", [("fp16", "sum"), ("bf16", "sum"), ("fp32", "prod"), ("int32", "max"),
                                      ("int8", "sum"), ("fp32", "min"), ("int16", "min")])
@pytest.mark.parametrize("k", [1, 2, 3, 8, 16, 32])
def test_reduce_k(gpu_thread, dtype, op, k):
    dt, o = DT[dtype], OPS[op]
    for count in (1, 4099, 300007):
        say("reduce_k", dtype, op, k, count)
        srcs = [gen(dt, count, 1000 + j, "prod" if op == "prod" else "default") for j in range(k)]
        want = oracle.reduce_k(srcs, dt, o)
        dev = [to_dev(s) for s in srcs]
        d_o = to_dev(np.zeros_like(srcs[0]))
        assert h.HcommGfxReduceKOnThread(gpu_thread, d_o.data_ptr(), [d.data_ptr() for d in dev], count, dt, o) == 0
        h.HcommGfxThreadSynchronize(gpu_thread)
        assert_same(from_dev(d_o, srcs[0]), want, dt)
        for j in range(k):
            assert np.array_equal(from_dev(dev[j], srcs[j]), srcs[j]), "input %d modified" % j


def test_notify_orders_two_threads(gpu_thread):
    """Record on thread A / wait on thread B: B's reduce sees A's copy (include/hcomm_primitives.h:181-191)."""
    code, (tb,) = h.HcommThreadAlloc(h.CommEngine.CPU_TS, 1, 1)
    assert code == 0
    try:
        count = 1 << 20
        x, y = gen(oracle.I32, count, 1), gen(oracle.I32, count, 2)
        d_x, d_y, d_t = to_dev(x), to_dev(y), to_dev(np.zeros_like(x))
        h.HcommGfxThreadSynchronize(gpu_thread)
        assert h.HcommThreadNotifyWaitOnThread(tb, 0, 10) == h.HcclResult.E_TIMEOUT   # no record issued yet
        assert h.HcommLocalCopyOnThread(gpu_thread, d_t.data_ptr(), d_x.data_ptr(), count * 4) == 0
        assert h.HcommThreadNotifyRecordOnThread(gpu_thread, tb, 0) == 0
        assert h.HcommThreadNotifyWaitOnThread(tb, 0, 10) == 0
        assert h.HcommThreadNotifyWaitOnThread(tb, 0, 10) == h.HcclResult.E_TIMEOUT   # that record is consumed
        assert h.HcommLocalReduceOnThread(tb, d_y.data_ptr(), d_t.data_ptr(), count, oracle.I32, oracle.SUM) == 0
        assert h.HcommGfxThreadSynchronize(tb) == 0
        assert_same(from_dev(d_y, y), (x + y), oracle.I32)
        assert h.HcommThreadNotifyWaitOnThread(tb, 1, 0) == h.HcclResult.E_PARA
    finally:
        h.HcommThreadFree([tb])


def test_mem_alloc_roundtrip(gpu_thread):
    code, p = h.HcommMemAlloc(1 << 20)
    assert code == 0 and p != 0 and p % 256 == 0
    src = np.random.default_rng(0).integers(0, 256, 1 << 20, dtype=np.uint8)
    d_src, d_back = to_dev(src), to_dev(np.zeros_like(src))
    assert h.HcommLocalCopyOnThread(gpu_thread, p, d_src.data_ptr(), src.size) == 0
    assert h.HcommLocalCopyOnThread(gpu_thread, d_back.data_ptr(), p, src.size) == 0
    h.HcommGfxThreadSynchronize(gpu_thread)
    assert np.array_equal(d_back.cpu().numpy(), src)
    assert h.HcommMemFree(p) == 0


def test_inter_rank_twins_and_descriptor_batch(gpu_thread):
    """Write / Read / WriteReduce / ReadReduce give the same bytes as their local twins, and a descriptor
    array submitted with HcommBatchTransferOnThread runs as one merged launch per kind."""
    dt, count, n = oracle.BF16, 40001, 6
    a = [gen(dt, count, 300 + i) for i in range(n)]
    b = [gen(dt, count, 400 + i) for i in range(n)]
    d_a, d_b = [to_dev(x) for x in a], [to_dev(x) for x in b]
    d_c = [to_dev(np.zeros_like(x)) for x in a]
    h.HcommGfxThreadSynchronize(gpu_thread)
    CH = 1
    assert h.HcommWriteReduceOnThread(gpu_thread, CH, d_a[0].data_ptr(), d_b[0].data_ptr(), count, dt, oracle.SUM) == 0
    assert h.HcommReadReduceOnThread(gpu_thread, CH, d_a[1].data_ptr(), d_b[1].data_ptr(), count, dt, oracle.MAX) == 0
    assert h.HcommWriteOnThread(gpu_thread, CH, d_c[0].data_ptr(), d_a[0].data_ptr(), count * 2) == 0
    assert h.HcommReadOnThread(gpu_thread, CH, d_c[1].data_ptr(), d_a[1].data_ptr(), count * 2) == 0
    descs = [h.desc_reduce(d_a[i].data_ptr(), d_b[i].data_ptr(), count, dt, oracle.SUM, read=(i % 2 == 0))
             for i in range(2, n)]
    descs += [h.desc_copy(d_c[i].data_ptr(), d_a[i].data_ptr(), count * 2, read=(i % 2 == 1)) for i in range(2, n)]
    h.HcommGfxLaunchLogClear(gpu_thread)
    assert h.HcommBatchTransferOnThread(gpu_thread, CH, descs) == 0
    assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
    assert [(r.kind, r.nseg) for r in h.launch_log(gpu_thread)] == [(h.Kernel.REDUCE2, n - 2), (h.Kernel.COPY, n - 2)]
    for i in range(n):
        want = oracle.reduce(a[i].copy(), b[i], dt, oracle.MAX if i == 1 else oracle.SUM)
        assert_same(from_dev(d_a[i], a[i]), want, dt, "a[%d]" % i)
        assert_same(from_dev(d_c[i], a[i]), want, dt, "c[%d]" % i)


def test_more_than_4gib_in_one_call(gpu_thread):
    """Lengths beyond 2^32 bytes / elements (the reference's API tests pass 4 GB and 4 GB + 1,
    ut_aicpu_ts_HcommLocalCopyOnThread.cc, ut_aicpu_ts_HcommLocalReduceOnThread.cc:71-89): 64-bit indexing end
    to end, checked on the GPU against torch."""
    import torch
    n = (1 << 32) + 5
    say("4GiB copy")
    src = torch.empty(n + 16, dtype=torch.int8, device="cuda")
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    src.random_(-100, 100, generator=g)
    dst = torch.zeros(n + 16, dtype=torch.int8, device="cuda")
    torch.cuda.synchronize()
    assert h.HcommLocalCopyOnThread(gpu_thread, dst.data_ptr(), src.data_ptr(), n) == 0
    assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
    assert torch.equal(dst[:n], src[:n]) and int(dst[n:].abs().max()) == 0
    say("4GiB reduce")
    want = (dst[n - 4096:n].to(torch.int16) + src[n - 4096:n].to(torch.int16)).to(torch.int8)   # wraps like int8
    head = (dst[:4096].to(torch.int16) + src[:4096].to(torch.int16)).to(torch.int8)
    mid0 = (1 << 32) - 2048
    mid = (dst[mid0:n].to(torch.int16) + src[mid0:n].to(torch.int16)).to(torch.int8)   # straddles 2^32
    torch.cuda.synchronize()   # torch computed the expectations on its own stream
    assert h.HcommLocalReduceOnThread(gpu_thread, dst.data_ptr(), src.data_ptr(), n, oracle.I8, oracle.SUM) == 0
    assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
    assert torch.equal(dst[:4096], head) and torch.equal(dst[n - 4096:n], want) and torch.equal(dst[mid0:n], mid)
    assert int(dst[n:].abs().max()) == 0, "reduce wrote past count"
    # whole-buffer check without a second 4 GiB temporary: dst == 2 * src in wrapping int8 arithmetic
    chunk = 1 << 28
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        assert torch.equal(dst[lo:hi], src[lo:hi] * 2), "chunk at %d" % lo
    del src, dst
    torch.cuda.empty_cache()


def test_batches_of_nearly_equal_segments(gpu_thread):
    """Batches whose segments differ a little in length take the (tile, segment) grid, as wide as the longest one:
    shorter segments leave workgroups with nothing to do, tails fall into different tiles.  A fixed-seed sample of
    segment counts, lengths around the tile boundaries, types and operations, reduces and copies, every buffer
    bit-exact against the oracle, and the launch records say which grid a batch took."""
    rng = np.random.default_rng(77)
    direct = h.HcommGfxSetDirectLaunches(1)   # the setting this test runs under (the other test module turns it off)
    h.HcommGfxSetDirectLaunches(direct)
    names = ["int8", "int16", "int32", "fp16", "fp32", "bf16"]
    bases = [100, 4096, 16384, 16384 * 3 + 5, 100000, 1 << 20]
    for case in range(40):
        nseg = int(rng.choice([1, 2, 3, 8, 9, 17, 64]))
        dtype = names[rng.integers(len(names))]
        op = ["sum", "max", "min"][rng.integers(3)]   # PROD is refused by the primitive unless opted in
        dt, o, unit = DT[dtype], OPS[op], UNIT[DT[dtype]]
        base = int(bases[rng.integers(len(bases))]) // unit + 1
        if nseg * base * unit > (48 << 20):
            base = (48 << 20) // (nseg * unit)
        counts = [max(1, base - int(rng.integers(0, base // 10 + 2))) for _ in range(nseg)]   # within 10 % of one another
        is_copy = bool(rng.integers(3) == 0)
        say("nearly equal", case, nseg, dtype, op, "copy" if is_copy else "reduce", counts[:4])
        dst = [gen(dt, c, 5000 + 2 * i) for i, c in enumerate(counts)]
        src = [gen(dt, c, 5001 + 2 * i) for i, c in enumerate(counts)]
        d_dst, d_src = [to_dev(x) for x in dst], [to_dev(x) for x in src]
        h.HcommGfxThreadSynchronize(gpu_thread)
        h.HcommGfxLaunchLogClear(gpu_thread)
        assert h.HcommBatchModeStart(b"rows") == 0
        for i, c in enumerate(counts):
            if is_copy:
                assert h.HcommLocalCopyOnThread(gpu_thread, d_dst[i].data_ptr(), d_src[i].data_ptr(), c * unit) == 0
            else:
                assert h.HcommLocalReduceOnThread(gpu_thread, d_dst[i].data_ptr(), d_src[i].data_ptr(), c, dt, o) == 0
        assert h.HcommBatchModeEnd(b"rows") == 0
        h.HcommGfxThreadSynchronize(gpu_thread)
        log = h.launch_log(gpu_thread)
        assert len(log) == 1 and log[0].nseg == nseg
        tiles = [(c * unit + 16383) // 16384 for c in counts]
        total, grid = sum(tiles), max(tiles) * nseg
        rows = max(tiles) if direct and (grid <= total + total // 8 or (total <= 512 and grid <= 2 * total)) else 0
        assert log[0].rows == rows and log[0].blocks == (grid if rows else total)
        for i in range(nseg):
            want = dst[i].copy()
            if is_copy:
                want = src[i].copy()
            else:
                oracle.reduce(want, src[i], dt, o)
            assert_same(from_dev(d_dst[i], dst[i]), want, dt, "case %d segment %d" % (case, i))
            assert np.array_equal(from_dev(d_src[i], src[i]), src[i]), "case %d: source %d modified" % (case, i)


@pytest.mark.parametrize("sizes", [
    [16384, 32768, 16385, 1, 49152],          # 1, 2, 2, 1, 3 tiles: a grid of 3 x 5 for 9 tiles
    [1, 1, 1],
    [16383] * 9 + [5],
    [65536, 65536 - 16, 65536 + 16, 65535],   # tails in the last tile, one tile further, and a byte short
    [3 * 16384 + 7] * 64,
])
def test_row_grid_leaves_short_segments_alone(gpu_thread, sizes):
    """Byte copies and int8 sums over segments of hand-picked lengths in one batch: the grid is as wide as the longest
    segment, so the workgroups past a shorter segment's last tile must touch nothing - every destination is checked
    together with the 64 guard bytes behind it."""
    guard = 64
    rng = np.random.default_rng(len(sizes))
    for reduce in (False, True):
        src = [rng.integers(-8, 9, n, dtype=np.int8) for n in sizes]
        dst = [rng.integers(-8, 9, n + guard, dtype=np.int8) for n in sizes]
        d_src, d_dst = [to_dev(x) for x in src], [to_dev(x) for x in dst]
        h.HcommGfxThreadSynchronize(gpu_thread)
        assert h.HcommBatchModeStart(b"short") == 0
        for i, n in enumerate(sizes):
            if reduce:
                assert h.HcommLocalReduceOnThread(gpu_thread, d_dst[i].data_ptr(), d_src[i].data_ptr(), n, oracle.I8, oracle.SUM) == 0
            else:
                assert h.HcommLocalCopyOnThread(gpu_thread, d_dst[i].data_ptr(), d_src[i].data_ptr(), n) == 0
        assert h.HcommBatchModeEnd(b"short") == 0
        h.HcommGfxThreadSynchronize(gpu_thread)
        for i, n in enumerate(sizes):
            want = dst[i].copy()
            want[:n] = (dst[i][:n].astype(np.int16) + src[i].astype(np.int16)).astype(np.int8) if reduce else src[i]
            assert np.array_equal(from_dev(d_dst[i], dst[i]), want), "segment %d of %r (%s)" % (i, sizes[:5], "reduce" if reduce else "copy")
