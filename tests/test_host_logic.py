"""Host-side behaviour of libhcomm_gfx.so that needs no GPU: exported symbols, argument checks in the
reference's order, batch-mode coalescing and schedule lowering, observed through a recorder thread (every
launch it would make is logged instead of executed - the role the mocked engine plays in the reference's
test/ut/framework/communicator/impl/independent_op/data_api/ut_aicpu_ts_HcommLocalReduceOnThread.cc)."""
import ctypes as C
import os
import re

import pytest

import hcomm_amd as h
from hcomm_amd import api as raw
from hcomm_amd import HcclResult as R, HcommDataType as DT, HcommReduceOp as OP

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture()
def rec():
    code, t = h.HcommGfxRecorderThreadAlloc()
    assert code == 0
    yield t
    h.HcommThreadFree([t])


def test_library_exports_every_declared_symbol():
    text = open(os.path.join(ROOT, "include", "hcomm_gfx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b(Hcomm\w+)\s*\(", text))
    assert {"HcommLocalCopyOnThread", "HcommLocalReduceOnThread", "HcommThreadAlloc", "HcommThreadFree",
            "HcommBatchModeStart", "HcommBatchModeEnd", "HcommMemAlloc", "HcommMemFree",
            "HcommGfxPlanCreate", "HcommGfxReduceKOnThread"} <= names
    for n in sorted(names):
        assert hasattr(h.lib, n), "libhcomm_gfx.so does not export " + n
    assert len(names) >= 27
    plugin = open(os.path.join(ROOT, "include", "hcomm_gfx_nic_plugin.h")).read()
    plugin = re.sub(r"/\*.*?\*/", "", plugin, flags=re.S)
    pnames = set(re.findall(r"\b(HcommNicPlugin\w+)\s*\(", plugin))
    assert pnames == {"HcommNicPluginGetInfo", "HcommNicPluginCreateEndpoint", "HcommNicPluginCreateChannel"}
    for n in sorted(pnames):
        assert hasattr(h.lib, n), "libhcomm_gfx.so does not export " + n


def test_enum_values_match_the_reference_headers():
    """include/hcomm_primitives.h:45-72, include/hccl/hccl_types.h:23-51."""
    assert (OP.SUM, OP.PROD, OP.MAX, OP.MIN, OP.RESERVED) == (0, 1, 2, 3, 255)
    assert (DT.INT8, DT.INT16, DT.INT32, DT.FP16, DT.FP32, DT.INT64, DT.UINT64, DT.UINT8, DT.UINT16, DT.UINT32,
            DT.FP64, DT.BFP16, DT.INT128, DT.HIF8, DT.FP8E4M3, DT.FP8E5M2, DT.FP8E8M0) == \
        (0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 14, 15, 16, 17)
    assert (R.SUCCESS, R.E_PARA, R.E_PTR, R.E_NOT_SUPPORT, R.E_TIMEOUT) == (0, 1, 2, 5, 9)
    sizes = [1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1]
    assert [h.HcommGfxDataTypeSize(i) for i in range(18)] == sizes and h.HcommGfxDataTypeSize(255) == 0


# ---- argument checks, in the reference's order (cpu_primitives_c_adpt.cc:58-130 and its unit tests) ------

DST, SRC = 0x100000, 0x200000


def test_local_reduce_checks(rec):
    f = h.HcommLocalReduceOnThread
    assert f(rec, DST, SRC, 1, DT.FP16, OP.SUM) == R.SUCCESS
    assert f(0, DST, SRC, 1, DT.FP16, OP.SUM) == R.E_PTR           # thread null
    assert f(rec, None, SRC, 1, DT.FP16, OP.SUM) == R.E_PTR        # dst null
    assert f(rec, DST, None, 1, DT.FP16, OP.SUM) == R.E_PTR        # src null
    # null pointers are reported before an unsupported type, an unsupported type before a null thread
    assert f(rec, None, SRC, 1, DT.FP64, OP.SUM) == R.E_PTR
    assert f(0, DST, SRC, 1, DT.FP64, OP.SUM) == R.E_PARA
    for bad in (DT.INT64, DT.UINT64, DT.UINT8, DT.UINT16, DT.UINT32, DT.FP64, DT.INT128, DT.HIF8, DT.FP8E4M3, 255, 13):
        assert f(rec, DST, SRC, 1, bad, OP.SUM) == R.E_PARA
    for good in (DT.INT8, DT.INT16, DT.INT32, DT.FP16, DT.FP32, DT.BFP16):
        for op in (OP.SUM, OP.MAX, OP.MIN):
            assert f(rec, DST, SRC, 1, good, op) == R.SUCCESS
        assert f(rec, DST, SRC, 1, good, OP.PROD) == R.E_PARA       # PROD only at collective level
        assert f(rec, DST, SRC, 1, good, OP.RESERVED) == R.E_PARA


def test_local_copy_checks(rec):
    f = h.HcommLocalCopyOnThread
    assert f(rec, DST, SRC, 1) == R.SUCCESS
    assert f(0, DST, SRC, 1) == R.E_PTR
    assert f(rec, None, SRC, 1) == R.E_PTR
    assert f(rec, DST, None, 1) == R.E_PTR


def test_counts_of_4gib_and_more_succeed(rec):
    """ut_aicpu_ts_HcommLocalReduceOnThread.cc:71-89, ut_aicpu_ts_HcommLocalCopyOnThread.cc (4 GB, 4 GB + 1)."""
    big, bigger = 0x100000000, 0x100000001
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommLocalReduceOnThread(rec, DST, SRC, big, DT.FP16, OP.SUM) == R.SUCCESS
    assert h.HcommLocalReduceOnThread(rec, DST, SRC, bigger, DT.FP16, OP.SUM) == R.SUCCESS
    assert h.HcommLocalCopyOnThread(rec, DST, SRC + (1 << 40), big) == R.SUCCESS
    assert h.HcommLocalCopyOnThread(rec, DST, SRC + (1 << 40), bigger) == R.SUCCESS
    log = h.launch_log(rec)
    assert [r.bytes for r in log] == [2 * big, 2 * bigger, big, bigger]    # no 32-bit truncation anywhere
    assert all(r.blocks > 0 for r in log)


def test_zero_length_and_self_copy_do_nothing(rec):
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommLocalReduceOnThread(rec, DST, SRC, 0, DT.FP32, OP.SUM) == R.SUCCESS
    assert h.HcommLocalCopyOnThread(rec, DST, SRC, 0) == R.SUCCESS
    assert h.HcommLocalCopyOnThread(rec, DST, DST, 4096) == R.SUCCESS
    assert h.launch_log(rec) == []


def test_thread_and_memory_argument_checks():
    assert raw._thread_alloc(h.CommEngine.CPU_TS, 1, (C.c_uint32 * 1)(0), None) == R.E_PTR
    assert raw._thread_alloc(h.CommEngine.CPU_TS, 1, None, (C.c_uint64 * 1)()) == R.E_PTR
    assert raw._thread_alloc(h.CommEngine.CPU_TS, 0, (C.c_uint32 * 1)(0), (C.c_uint64 * 1)()) == R.E_PARA
    assert raw._thread_free(None, 1) == R.E_PTR
    assert raw._thread_free_stream(None, 1) == R.E_PTR
    assert raw._thread_free_stream((C.c_uint64 * 1)(0), 0) == R.E_PARA
    assert raw._thread_alloc_stream(h.CommEngine.CPU_TS, None, 0, None) == R.E_PTR
    assert raw._mem_alloc(None, 16) == R.E_PTR
    assert raw._mem_alloc(C.byref(C.c_void_p()), 0) == R.E_PARA
    assert h.HcommMemFree(None) == R.E_PTR
    assert h.HcommGfxThreadSynchronize(0) == R.E_PTR
    assert h.HcommThreadFree([12345]) == R.E_NOT_FOUND             # not a live handle: refused, never dereferenced
    assert h.HcommLocalCopyOnThread(12345, DST, SRC, 1) == R.E_PTR


def test_notify_argument_checks(rec):
    assert h.HcommThreadNotifyRecordOnThread(0, rec, 0) == R.E_PTR
    assert h.HcommThreadNotifyRecordOnThread(rec, 0, 0) == R.E_PTR
    assert h.HcommThreadNotifyRecordOnThread(rec, rec, 32) == R.E_PARA  # a recorder thread has 32 notify slots
    assert h.HcommThreadNotifyWaitOnThread(0, 0, 1) == R.E_PTR
    assert h.HcommThreadNotifyWaitOnThread(rec, 32, 1) == R.E_PARA


def test_notify_wait_needs_a_record_issued_before_it(rec):
    """A notify is an event on a stream: a wait can only follow a record that has been issued.  The wait that finds
    none is the one the reference would time out on (include/hcomm_primitives.h:191): HCCL_E_TIMEOUT, at once."""
    code, other = h.HcommGfxRecorderThreadAlloc()
    assert code == 0
    try:
        assert h.HcommThreadNotifyWaitOnThread(rec, 0, 10) == R.E_TIMEOUT            # nothing recorded yet
        assert h.HcommThreadNotifyRecordOnThread(other, rec, 0) == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThread(rec, 1, 10) == R.E_TIMEOUT            # the record went to slot 0
        assert h.HcommThreadNotifyWaitOnThread(rec, 0, 10) == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThread(rec, 0, 10) == R.E_TIMEOUT            # one record, one wait
        for _ in range(3):
            assert h.HcommThreadNotifyRecordOnThread(other, rec, 1) == R.SUCCESS
        for _ in range(3):
            assert h.HcommThreadNotifyWaitOnThreadWithDefaultTimeout(rec, 1) == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThreadWithDefaultTimeout(rec, 1) == R.E_TIMEOUT
    finally:
        h.HcommThreadFree([other])


def _fake(n, base):
    return [base + r * (1 << 26) for r in range(n)]


@pytest.mark.parametrize("alg,n,count,dt", [
    (h.Alg.ALLREDUCE_RING, 8, 1 << 20, h.HcommDataType.BFP16),
    (h.Alg.ALLREDUCE_RHD, 16, 1 << 18, h.HcommDataType.INT32),
    (h.Alg.ALLREDUCE_RHD, 6, 100003, h.HcommDataType.FP32),
    (h.Alg.ALLREDUCE_MESH_ONESHOT, 8, 2048, h.HcommDataType.FP16),
    (h.Alg.ALLREDUCE_NHR, 5, 70001, h.HcommDataType.BFP16),
    (h.Alg.REDUCE_SCATTER_RING, 7, 1000003, h.HcommDataType.FP32),
    (h.Alg.REDUCE_SCATTER_MESH, 7, 999, h.HcommDataType.INT32),
])
def test_one_batch_over_a_thread_per_rank_with_notifies_is_the_plans_launches(alg, n, count, dt):
    """The reference hands a batch over ALL its threads, notifies included, to one task graph (launch_context.cc:16-44
    CommTaskLaunch(threads, threadNum)).  Here HcommBatchModeEnd resolves the records and waits on the host: a
    collective given as rank r's calls on thread r, posts and waits between the steps, all inside one Start / End
    pair, comes out as the launches of the step-wise plan - every rank of a step in one launch - on the first
    thread of the batch, and no record is left pending."""
    from hcomm_amd import caller
    recs = [h.HcommGfxRecorderThreadAlloc()[1] for _ in range(n)]
    try:
        i, o = _fake(n, 1 << 40), _fake(n, 1 << 41)
        rp = caller.Replay(h.schedule_emit(alg, n, count, dt), {0: i, 1: o}, dt, 0)
        code, st = rp.run_on_threads_batched(recs)
        assert code == 0 and st.notifies >= 2 * (n - 1)
        plan = h.Plan(alg, h.Lowering.STEPWISE, i, o, count, dt, 0)
        key = lambda l: (l.kind, l.nseg, l.bytes, l.dtype, l.op)
        assert [key(l) for l in h.launch_log(recs[0])] == [key(l) for l in plan.launches()]
        assert all(not h.launch_log(t) for t in recs[1:])
        for t in recs:
            for q in range(n):
                assert h.HcommThreadNotifyWaitOnThread(t, q, 0) == R.E_TIMEOUT
    finally:
        h.HcommThreadFree(recs)


def test_notifies_inside_a_batch_are_resolved_at_its_end(rec):
    """Records and waits between HcommBatchModeStart and End are steps of their threads' sequences: End orders the
    copies and reduces by them.  A wait may come before its record in call order (another thread's record further
    down); a wait nothing satisfies fails the whole batch with HCCL_E_TIMEOUT and submits nothing; a record no wait
    of the batch consumes - and one issued before the batch - stay good for a wait outside it."""
    code, other = h.HcommGfxRecorderThreadAlloc()
    assert code == 0
    A, B, C_ = 1 << 40, 1 << 41, 1 << 42
    try:
        # other: B <- A, then posts; rec: waits, then C <- B.  Called in the "wrong" order: rec first.
        assert h.HcommBatchModeStart(b"b") == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThread(rec, 3, 10) == R.SUCCESS
        assert h.HcommLocalCopyOnThread(rec, C_, B, 8192) == R.SUCCESS
        assert h.HcommLocalCopyOnThread(other, B, A, 4096) == R.SUCCESS
        assert h.HcommThreadNotifyRecordOnThread(other, rec, 3) == R.SUCCESS
        assert h.HcommThreadNotifyRecordOnThread(other, rec, 4) == R.SUCCESS   # nobody in the batch waits for this one
        assert h.HcommBatchModeEnd(b"b") == R.SUCCESS
        log = h.launch_log(rec)                                                # the first thread of the batch issues all
        # B<-A (4 KiB) before C<-B (8 KiB), and apart: C<-B reads what B<-A writes
        assert [(l.kind, l.nseg, l.bytes) for l in log] == [(0, 1, 4096), (0, 1, 8192)]
        assert not h.launch_log(other)
        assert h.HcommThreadNotifyWaitOnThread(rec, 3, 0) == R.E_TIMEOUT       # consumed inside the batch
        assert h.HcommThreadNotifyWaitOnThread(rec, 4, 0) == R.SUCCESS         # left over from the batch
        # a record issued before the batch satisfies a wait inside it
        h.HcommGfxLaunchLogClear(rec)
        assert h.HcommThreadNotifyRecordOnThread(other, rec, 5) == R.SUCCESS
        assert h.HcommBatchModeStart(b"b") == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThread(rec, 5, 10) == R.SUCCESS
        assert h.HcommLocalCopyOnThread(rec, C_, B, 4096) == R.SUCCESS
        assert h.HcommBatchModeEnd(b"b") == R.SUCCESS
        assert len(h.launch_log(rec)) == 1
        assert h.HcommThreadNotifyWaitOnThread(rec, 5, 0) == R.E_TIMEOUT
        # two threads waiting for each other before either posts: nothing can run
        h.HcommGfxLaunchLogClear(rec)
        assert h.HcommThreadNotifyRecordOnThread(other, rec, 6) == R.SUCCESS   # an earlier record the failed batch takes ...
        assert h.HcommBatchModeStart(b"b") == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThread(rec, 6, 10) == R.SUCCESS
        assert h.HcommLocalCopyOnThread(rec, C_, B, 4096) == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThread(rec, 0, 10) == R.SUCCESS
        assert h.HcommThreadNotifyRecordOnThread(rec, other, 0) == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThread(other, 0, 10) == R.SUCCESS
        assert h.HcommThreadNotifyRecordOnThread(other, rec, 0) == R.SUCCESS
        assert h.HcommBatchModeEnd(b"b") == R.E_TIMEOUT
        assert not h.launch_log(rec) and not h.launch_log(other)
        assert h.HcommThreadNotifyWaitOnThread(rec, 6, 0) == R.SUCCESS         # ... and hands back
        assert h.HcommThreadNotifyWaitOnThread(rec, 0, 0) == R.E_TIMEOUT
        assert h.HcommThreadNotifyWaitOnThread(other, 0, 0) == R.E_TIMEOUT
        # the threads are free again
        assert h.HcommLocalCopyOnThread(other, B, A, 4096) == R.SUCCESS
        # slot numbers are checked when the call is made
        assert h.HcommBatchModeStart(b"b") == R.SUCCESS
        assert h.HcommThreadNotifyWaitOnThread(rec, 32, 10) == R.E_PARA
        assert h.HcommThreadNotifyRecordOnThread(other, rec, 32) == R.E_PARA
        assert h.HcommBatchModeEnd(b"b") == R.SUCCESS
    finally:
        h.HcommThreadFree([other])


def test_notify_wait_sits_for_a_record_another_host_thread_issues_late(rec):
    """Callers that drive each thread from a host thread of its own cannot order a wait after its record: the wait
    sits on the host (at most min(timeOut, HCOMM_GFX_NOTIFY_HOST_WAIT_MS)) until the record has been issued; a
    timeOut of 0 seconds does not sit at all."""
    import threading
    import time
    code, other = h.HcommGfxRecorderThreadAlloc()
    assert code == 0
    try:
        t0 = time.perf_counter()
        assert h.HcommThreadNotifyWaitOnThread(rec, 0, 0) == R.E_TIMEOUT
        assert time.perf_counter() - t0 < 0.05
        late = threading.Timer(0.02, lambda: h.HcommThreadNotifyRecordOnThread(other, rec, 0))
        late.start()
        assert h.HcommThreadNotifyWaitOnThread(rec, 0, 10) == R.SUCCESS      # ctypes releases the GIL during the call
        late.join()
        assert h.HcommThreadNotifyWaitOnThread(rec, 0, 0) == R.E_TIMEOUT     # that record is consumed
    finally:
        h.HcommThreadFree([other])


def test_a_thread_in_another_host_threads_batch_takes_nothing(rec):
    """Between HcommBatchModeStart and End of one host thread, the threads it recorded on refuse every other host
    thread - batching or not, primitives, k-way reduce, plans and the entry point that allocates nothing alike - and
    a plan or that entry point is refused inside the caller's own batch, where its launches would run ahead of what
    the batch recorded (launch_context.cc:139-174: everything between Start and End is submitted at End)."""
    import threading
    ins = [0x1000000 * (r + 1) for r in range(4)]
    outs = [(1 << 36) + 0x1000000 * (r + 1) for r in range(4)]
    plan = h.Plan(h.Alg.ALLREDUCE_RING, h.Lowering.STEPWISE, ins, outs, 4096, DT.FP32, OP.SUM)
    seen = {}

    def other_host_thread():
        seen["copy"] = h.HcommLocalCopyOnThread(rec, DST, SRC, 64)
        seen["reduce_k"] = h.HcommGfxReduceKOnThread(rec, DST, [SRC, SRC + 4096], 16, DT.FP32, OP.SUM)
        seen["plan"] = plan.run(rec)
        seen["no_alloc"] = h.HcommGfxAllReduceLocalReduceNoAlloc(rec, ins, outs, 4096, DT.FP32, OP.SUM)
        h.HcommBatchModeStart(b"theirs")
        seen["batched_copy"] = h.HcommLocalCopyOnThread(rec, DST, SRC, 64)
        seen["end"] = h.HcommBatchModeEnd(b"theirs")

    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommBatchModeStart(b"mine") == R.SUCCESS
    try:
        assert h.HcommLocalCopyOnThread(rec, DST, SRC, 64) == R.SUCCESS       # rec now belongs to this batch
        assert plan.run(rec) == R.E_NOT_SUPPORT
        assert h.HcommGfxAllReduceLocalReduceNoAlloc(rec, ins, outs, 4096, DT.FP32, OP.SUM) == R.E_NOT_SUPPORT
        th = threading.Thread(target=other_host_thread)
        th.start()
        th.join()
        assert seen == {"copy": R.E_UNAVAIL, "reduce_k": R.E_UNAVAIL, "plan": R.E_UNAVAIL, "no_alloc": R.E_UNAVAIL,
                        "batched_copy": R.E_UNAVAIL, "end": R.SUCCESS}
        assert h.launch_log(rec) == []                                         # nothing ran ahead of the batch
    finally:
        assert h.HcommBatchModeEnd(b"mine") == R.SUCCESS
    assert len(h.launch_log(rec)) == 1
    assert plan.run(rec) == R.SUCCESS                                          # free again after End
    plan.destroy()


@pytest.mark.parametrize("alg,n,count,dt", [(h.Alg.ALLREDUCE_RING, 8, 1 << 20, DT.BFP16), (h.Alg.ALLREDUCE_RHD, 6, 100003, DT.FP32),
                                            (h.Alg.ALLREDUCE_MESH_ONESHOT, 8, 2048, DT.FP16), (h.Alg.REDUCE_SCATTER_RING, 7, 1000003, DT.INT8),
                                            (h.Alg.REDUCE_SCATTER_MESH, 4, 4096, DT.FP16)])
def test_a_caller_that_batches_each_step_gets_the_plans_launches(rec, alg, n, count, dt):
    """The reference's own boundary, driven the way its caller drives it (hcomm_amd/csrc/hg_caller.c: one
    HcommBatchModeStart / End pair per schedule step, every rank's HcommLocalCopy/ReduceOnThread call between them):
    the launches are those of the step-wise plan - same kernels, segments, bytes and grids, in the same order.  (A plan
    may do better where two consecutive steps are independent - the own-slice copy and the first gather step of NHR share
    a launch there - which a caller that ends its batch at every step cannot.)"""
    from hcomm_amd import caller
    scatter = alg == h.Alg.REDUCE_SCATTER_MESH
    i, o = ptrs(n, count * h.DTYPE_SIZE[dt] * (n if scatter else 1), base=1 << 40)
    plan = h.Plan(alg, h.Lowering.STEPWISE, i, None if alg == h.Alg.REDUCE_SCATTER_RING else o, count, dt, OP.SUM)
    want = _launch_tuples(plan.launches())
    plan.destroy()
    ops = h.schedule_emit(alg, n, count, dt)
    replay = caller.Replay(ops, {0: i, 1: o}, dt, OP.SUM)
    h.HcommGfxLaunchLogClear(rec)
    code, st = replay.run_batched(rec)
    assert code == R.SUCCESS
    assert (st.batches, st.calls) == (replay.steps, len(ops))
    assert _launch_tuples(h.launch_log(rec)) == want


def test_a_caller_with_one_thread_per_rank_posts_to_the_peers_it_exchanges_with():
    """Rank r's calls on thread r, nothing batched: between the steps of a ring every thread waits for the rank it
    reads (data) and for the rank that read it (acknowledgement) - reduce_scatter_ring.cc:211-217,254-272 - and for
    nobody else; thread 0 forks and joins the others."""
    from hcomm_amd import caller
    n, count, dt = 8, 1 << 16, DT.FP32
    recs = []
    for _ in range(n):
        code, t = h.HcommGfxRecorderThreadAlloc()
        assert code == 0
        recs.append(t)
    try:
        i, o = ptrs(n, count * 4, base=1 << 40)
        ops = h.schedule_emit(h.Alg.ALLREDUCE_RING, n, count, dt)
        code, st = caller.Replay(ops, {0: i, 1: o}, dt, OP.SUM).run_on_threads(recs)
        assert code == R.SUCCESS
        steps = 2 * (n - 1) + 1
        assert (st.batches, st.calls) == (steps, len(ops))
        # fork and join: n - 1 each.  Step 0 needs nobody.  A reduce-scatter or all-gather step after the first of its
        # stage: two waits per rank (data from r - 1, acknowledgement from r + 1).  The own-slice copy between the
        # stages reads no peer (acknowledgement only) and the first all-gather step follows a step in which nobody
        # read rank r (data only): one wait per rank each.
        assert st.notifies == 2 * (n - 1) + 2 * n * (steps - 3) + 2 * n
        for r in range(n):                       # every rank's thread got its own 15 launches, one segment each
            log = h.launch_log(recs[r])
            assert len(log) == steps and all(x.nseg == 1 for x in log)
        # every record was consumed by its wait
        for r in range(n):
            for q in range(n):
                assert h.HcommThreadNotifyWaitOnThread(recs[r], q, 0) == R.E_TIMEOUT
        # the same with a host thread per rank, five times over: waits that reach the library before their record sit
        # until it is issued; same calls, same posts and waits, same launches on every rank's thread
        for r in range(n):
            h.HcommGfxLaunchLogClear(recs[r])
        for it in range(5):
            code, st2 = caller.Replay(ops, {0: i, 1: o}, dt, OP.SUM).run_on_host_threads(recs)
            assert code == R.SUCCESS
            assert (st2.batches, st2.calls, st2.notifies) == (steps, len(ops), st.notifies)
        for r in range(n):
            assert len(h.launch_log(recs[r])) == 5 * steps
            for q in range(n):
                assert h.HcommThreadNotifyWaitOnThread(recs[r], q, 0) == R.E_TIMEOUT
    finally:
        caller.pool_shutdown()
        h.HcommThreadFree(recs)


def test_timeouts_fences_and_non_blocking_twins(rec):
    """include/hcomm_primitives.h:317-318,370-371,534,542,559,567,585,593 with the host adapter's checks."""
    nan, CH = float("nan"), 0x77
    assert h.HcommSetNotifyWaitTimeOut(nan) == R.E_PARA
    assert h.HcommSetNotifyWaitTimeOut(-1.0) == R.E_PARA
    assert h.HcommSetNotifyWaitTimeOut(5e9) == R.E_PARA
    assert h.HcommSetNotifyWaitTimeOut(30.5) == R.SUCCESS
    assert h.HcommThreadResAcquireTimeOut(1.0) == R.E_NOT_SUPPORT
    assert h.HcommThreadNotifyWaitOnThreadWithDefaultTimeout(rec, 32) == R.E_PARA      # the recorder has 32 notify slots
    assert h.HcommThreadNotifyWaitOnThreadWithDefaultTimeout(12345, 0) == R.E_PTR
    assert h.HcommFenceOnThread(rec) == R.SUCCESS and h.HcommFenceOnThread(12345) == R.E_PTR
    assert h.HcommChannelFenceOnThread(rec, CH) == R.SUCCESS and h.HcommChannelFenceOnThread(rec, 0) == R.E_PTR
    assert h.HcommChannelDrainOnThread(rec, CH) == R.SUCCESS and h.HcommChannelDrainOnThread(rec, 0) == R.E_PTR
    assert h.HcommChannelDrainOnThread(12345, CH) == R.E_PTR
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommWriteNbiOnThread(rec, CH, DST, SRC, 4096) == 0
    assert h.HcommReadNbiOnThread(rec, CH, DST, SRC, 8192) == 0
    assert h.HcommWriteNbiOnThread(rec, 0, DST, SRC, 4096) == R.E_PTR
    assert [(r.kind, r.bytes) for r in h.launch_log(rec)] == [(h.Kernel.COPY, 4096), (h.Kernel.COPY, 8192)]


def test_inter_rank_twins_checks_and_launches(rec):
    """HcommWrite/Read[Reduce]OnThread: same arithmetic with a channel argument
    (cpu_primitives_c_adpt.cc:284-318,332-384,490-565)."""
    CH = 0x77
    for f in (h.HcommWriteOnThread, h.HcommReadOnThread):
        assert f(rec, CH, DST, SRC, 4096) == R.SUCCESS
        assert f(rec, CH, None, SRC, 4096) == R.E_PTR
        assert f(rec, CH, DST, None, 4096) == R.E_PTR
        assert f(0, CH, DST, SRC, 4096) == R.E_PTR
        assert f(rec, 0, DST, SRC, 4096) == R.E_PTR
    for f in (h.HcommWriteReduceOnThread, h.HcommReadReduceOnThread):
        assert f(rec, CH, DST, SRC, 1024, DT.FP16, OP.SUM) == R.SUCCESS
        assert f(rec, CH, None, SRC, 1024, DT.FP16, OP.SUM) == R.E_PTR
        assert f(rec, CH, DST, SRC, 1024, DT.FP64, OP.SUM) == R.E_PARA
        assert f(rec, CH, DST, SRC, 1024, DT.FP16, OP.PROD) == R.E_PARA
        assert f(0, CH, DST, SRC, 1024, DT.FP64, OP.SUM) == R.E_PARA     # type check precedes the thread check
        assert f(0, CH, DST, SRC, 1024, DT.FP16, OP.SUM) == R.E_PTR
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommBatchModeStart(None) == 0
    for r in range(4):
        assert h.HcommReadReduceOnThread(rec, CH, DST + r * 65536, SRC + r * 65536, 1024, DT.BFP16, OP.MAX) == 0
    assert h.HcommBatchModeEnd(None) == 0
    assert [(x.kind, x.nseg, x.op) for x in h.launch_log(rec)] == [(h.Kernel.REDUCE2, 4, OP.MAX)]


def test_batch_transfer_descriptors(rec):
    """HcommBatchTransferDesc[] is one batch: independent descriptors share a launch, order is kept."""
    CH, K = 5, 65536
    descs = [h.desc_reduce(DST + r * K, SRC + r * K, 1024, DT.FP32, OP.SUM, read=True) for r in range(8)]
    descs += [h.desc_copy(DST + (20 + r) * K, DST + r * K, 4096) for r in range(8)]   # depend on the reduces
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommBatchTransferOnThread(rec, CH, descs) == R.SUCCESS
    assert [(x.kind, x.nseg) for x in h.launch_log(rec)] == [(h.Kernel.REDUCE2, 8), (h.Kernel.COPY, 8)]
    assert h.HcommBatchTransferOnThread(rec, CH, []) == R.SUCCESS
    assert h.HcommBatchTransferOnThread(0, CH, descs) == R.E_PTR
    assert h.HcommBatchTransferOnThread(rec, 0, descs) == R.E_PTR
    assert raw._batch_transfer(rec, CH, None, 3) == R.E_PTR
    h.HcommGfxLaunchLogClear(rec)
    bad = h.desc_reduce(DST, SRC, 16, DT.FP64, OP.SUM)
    assert h.HcommBatchTransferOnThread(rec, CH, descs[:2] + [bad]) == R.E_PARA
    notify = h.BatchTransferDesc()
    notify.transType = h.TransferType.NOTIFY_RECORD
    assert h.HcommBatchTransferOnThread(rec, CH, descs[:2] + [notify]) == R.E_NOT_SUPPORT
    null = h.desc_copy(0, SRC, 16)
    assert h.HcommBatchTransferOnThread(rec, CH, [null]) == R.E_PTR
    assert h.launch_log(rec) == []                     # validated as a whole before anything is enqueued
    import ctypes
    assert C.sizeof(h.BatchTransferDesc) == 64    # include/hcomm_primitives.h:91-131


def test_local_reduce_plan_needs_scratch_and_power_of_two(rec):
    i, o = ptrs(8, 1 << 22)
    sc, _ = ptrs(8, 1 << 23, base=0x90000000)
    count = 1 << 20
    assert h.scratch_bytes(h.Alg.ALLREDUCE_LOCAL_REDUCE, 8, count, DT.FP32) == 8 * (count * 4 // 8)
    assert h.scratch_bytes(h.Alg.ALLREDUCE_RING, 8, count, DT.FP32) == 0
    with pytest.raises(h.HcommError) as e:
        h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.STEPWISE, i, o, count, DT.FP32, OP.SUM)
    assert e.value.code == R.E_PTR                                   # no communication buffers given
    with pytest.raises(h.HcommError) as e:
        h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.STEPWISE, i[:6], o[:6], count, DT.FP32, OP.SUM, 0, sc[:6])
    assert e.value.code == R.E_PARA                                  # 6 ranks
    with pytest.raises(h.HcommError) as e:
        h.Plan(h.Alg.ALLREDUCE_DOUBLING, h.Lowering.FUSED, i, o, count, DT.FP32, OP.SUM)
    assert e.value.code == R.E_NOT_SUPPORT                           # no single-launch lowering
    p = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, i, o, count, DT.FP32, OP.SUM)   # user buffers only
    assert [(r.kind, r.nseg) for r in p.launches()] == [(h.Kernel.TREE, 8)]
    p.destroy()
    p = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.STEPWISE, i, o, count, DT.FP32, OP.SUM, 0, sc)
    # own copy | 6 gather rounds merged | neighbour reduce | fold + 2 halving rounds | own gather + 7 rounds merged
    kinds = [(r.kind, r.nseg) for r in p.launches()]
    assert kinds[0] == (h.Kernel.COPY, 56) and sum(ns for k, ns in kinds if k == h.Kernel.COPY) == 8 + 48 + 8 + 56
    assert sum(ns for k, ns in kinds if k == h.Kernel.REDUCE2) == 8 + 8 * 3 + 8 * 2 + 8 * 1
    assert p.info.movedBytes == p.info.algorithmicBytes
    p.destroy()


def test_strided_plan_checks():
    i, o = ptrs(4, 1 << 20)
    p = h.Plan(h.Alg.REDUCE_SCATTER_MESH, h.Lowering.FUSED, i, o, 1000, DT.FP32, OP.SUM, stride=1500)
    assert p.info.launches == 1
    p.destroy()
    for alg, stride, code in ((h.Alg.REDUCE_SCATTER_MESH, 999, R.E_PARA), (h.Alg.ALLREDUCE_RING, 1500, R.E_PARA)):
        with pytest.raises(h.HcommError) as e:
            h.Plan(alg, h.Lowering.STEPWISE, i, o, 1000, DT.FP32, OP.SUM, stride=stride)
        assert e.value.code == code


# ---- batch mode --------------------------------------------------------------------------------------------

def test_batch_mode_state_machine(rec):
    assert h.HcommBatchModeEnd(b"x") == R.E_PARA                   # End without Start
    assert h.HcommBatchModeStart(b"x") == R.SUCCESS
    assert h.HcommBatchModeStart(b"x") == R.E_PARA                 # nested Start
    assert h.HcommBatchModeEnd(b"x") == R.SUCCESS
    assert h.HcommBatchModeStart(None) == R.SUCCESS                # default tag
    assert h.HcommBatchModeEnd(None) == R.SUCCESS


def test_batch_mode_records_then_merges(rec):
    mib = 1 << 20
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommBatchModeStart(b"step0") == 0
    for r in range(8):   # eight independent reduces: one launch
        assert h.HcommLocalReduceOnThread(rec, DST + 2 * r * mib, DST + (2 * r + 1) * mib, mib // 2, DT.BFP16, OP.SUM) == 0
    assert h.launch_log(rec) == []                                 # nothing is submitted before End
    assert h.HcommBatchModeEnd(b"step0") == 0
    log = h.launch_log(rec)
    assert [(r.kind, r.nseg, r.bytes, r.dtype, r.op) for r in log] == [(h.Kernel.REDUCE2, 8, 8 * mib, DT.BFP16, OP.SUM)]


def test_batch_mode_splits_on_conflict_kind_type_and_capacity(rec):
    mib = 1 << 20
    A, B, Cc, D = DST, DST + 4 * mib, DST + 8 * mib, DST + 12 * mib

    def run(calls):
        h.HcommGfxLaunchLogClear(rec)
        assert h.HcommBatchModeStart(None) == 0
        for c in calls:
            assert c() == 0
        assert h.HcommBatchModeEnd(None) == 0
        return [(r.kind, r.nseg) for r in h.launch_log(rec)]

    red = lambda d, s, dt=DT.FP32, op=OP.SUM: (lambda: h.HcommLocalReduceOnThread(rec, d, s, mib // 4, dt, op))
    cp = lambda d, s: (lambda: h.HcommLocalCopyOnThread(rec, d, s, mib))
    K = h.Kernel
    assert run([red(A, B), red(Cc, D)]) == [(K.REDUCE2, 2)]
    assert run([red(A, B), red(Cc, A)]) == [(K.REDUCE2, 1), (K.REDUCE2, 1)]      # reads what the first writes
    assert run([red(A, B), red(B, Cc)]) == [(K.REDUCE2, 1), (K.REDUCE2, 1)]      # writes what the first reads
    assert run([red(A, B), red(A + mib // 2, D)]) == [(K.REDUCE2, 1), (K.REDUCE2, 1)]  # overlapping destinations
    assert run([red(A, B), red(Cc, B)]) == [(K.REDUCE2, 2)]                      # a shared source is fine
    assert run([red(A, B), cp(Cc, D)]) == [(K.REDUCE2, 1), (K.COPY, 1)]          # different kernels
    assert run([red(A, B), red(Cc, D, DT.INT32)]) == [(K.REDUCE2, 1), (K.REDUCE2, 1)]
    assert run([red(A, B), red(Cc, D, DT.FP32, OP.MAX)]) == [(K.REDUCE2, 1), (K.REDUCE2, 1)]
    assert run([cp(A, B), cp(Cc, D), cp(D + 2 * mib, A)]) == [(K.COPY, 2), (K.COPY, 1)]
    # both operands 4 bytes past a 16-byte boundary: 12 bytes element-wise, the rest at full width
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommLocalReduceOnThread(rec, A + 4, B + 4, mib // 4, DT.FP32, OP.SUM) == 0
    assert [(r.kind, r.bytes) for r in h.launch_log(rec)] == [(K.BYTEWISE, 12), (K.REDUCE2, mib - 12)]
    assert run([red(A + 4, B + 8)]) == [(K.BYTEWISE, 1)]                          # different misalignment
    small = lambda: h.HcommLocalReduceOnThread(rec, A + 4, B + 4, 1000, DT.FP32, OP.SUM)
    assert run([small]) == [(K.BYTEWISE, 1)]                                      # too small to be worth two launches
    many = [cp(DST + (2 * i) * mib, DST + (2 * i + 1) * mib) for i in range(134)]
    assert run(many) == [(K.COPY, 64), (K.COPY, 64), (K.COPY, 6)]                 # 64 segments per launch


def test_batch_mode_spans_several_threads(rec):
    code, other = h.HcommGfxRecorderThreadAlloc()
    assert code == 0
    for t in (rec, other):
        h.HcommGfxLaunchLogClear(t)
    assert h.HcommBatchModeStart(b"two") == 0
    assert h.HcommLocalCopyOnThread(rec, DST, SRC, 4096) == 0
    assert h.HcommLocalCopyOnThread(other, DST, SRC, 8192) == 0
    assert h.HcommLocalCopyOnThread(rec, DST + 65536, SRC + 65536, 4096) == 0
    assert h.HcommBatchModeEnd(b"two") == 0
    assert [(r.nseg, r.bytes) for r in h.launch_log(rec)] == [(2, 8192)]
    assert [(r.nseg, r.bytes) for r in h.launch_log(other)] == [(1, 8192)]
    h.HcommThreadFree([other])


def test_thread_freed_inside_a_batch_is_dropped_from_it(rec):
    code, other = h.HcommGfxRecorderThreadAlloc()
    assert code == 0
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommBatchModeStart(b"gone") == 0
    assert h.HcommLocalCopyOnThread(other, DST, SRC, 8192) == 0
    assert h.HcommLocalCopyOnThread(rec, DST, SRC, 4096) == 0
    assert h.HcommThreadFree([other]) == 0
    assert h.HcommBatchModeEnd(b"gone") == 0          # the freed thread's operations went with it
    assert [(r.nseg, r.bytes) for r in h.launch_log(rec)] == [(1, 4096)]
    assert h.HcommLocalCopyOnThread(other, DST, SRC, 8192) == R.E_PTR


def test_reduce_k_checks(rec):
    f = h.HcommGfxReduceKOnThread
    assert f(rec, DST, [SRC, SRC + 4096], 100, DT.FP16, OP.SUM) == R.SUCCESS
    assert f(rec, DST, [SRC], 100, DT.FP32, OP.PROD) == R.SUCCESS            # PROD allowed here
    assert f(rec, DST, [SRC], 100, DT.INT16, OP.PROD) == R.E_PARA            # not for int16 (param_check.cc:327-343)
    assert f(rec, DST, [SRC], 100, DT.BFP16, OP.PROD) == R.E_PARA            # nor for bf16
    assert f(rec, DST, [SRC], 100, DT.FP16, OP.PROD) == R.SUCCESS
    assert f(rec, None, [SRC], 100, DT.FP16, OP.SUM) == R.E_PTR
    assert f(rec, DST, [SRC, 0], 100, DT.FP16, OP.SUM) == R.E_PTR
    assert f(rec, DST, [], 100, DT.FP16, OP.SUM) == R.E_PARA
    assert f(rec, DST, [SRC] * 33, 100, DT.FP16, OP.SUM) == R.E_PARA
    assert f(0, DST, [SRC], 100, DT.FP16, OP.SUM) == R.E_PTR
    h.HcommGfxLaunchLogClear(rec)
    assert f(rec, DST, [SRC + i * 4096 for i in range(8)], 2048, DT.FP16, OP.SUM) == 0
    assert [(r.kind, r.nseg, r.bytes) for r in h.launch_log(rec)] == [(h.Kernel.CHAIN, 1, 4096)]
    h.HcommGfxLaunchLogClear(rec)
    assert f(rec, DST + 2, [SRC, SRC + 4096, SRC + 8192], 100, DT.FP16, OP.SUM) == 0   # unaligned: copy + 2 reduces
    assert [r.kind for r in h.launch_log(rec)] == [h.Kernel.BYTEWISE] * 3


# ---- plans ---------------------------------------------------------------------------------------------------

def ptrs(n, size, base=0x10000000):
    stride = (size + 255) // 256 * 256 + 256
    return [base + i * stride for i in range(n)], [base + (n + i) * stride for i in range(n)]


def test_plan_argument_checks():
    i, o = ptrs(4, 4096)
    mk = lambda **k: h.Plan(k.get("alg", h.Alg.ALLREDUCE_RING), k.get("low", h.Lowering.STEPWISE), k.get("i", i),
                            k.get("o", o), 1024, k.get("dt", DT.FP32), k.get("op", OP.SUM))
    mk().destroy()
    for kwargs, code in (({"dt": DT.FP64}, R.E_PARA), ({"op": OP.RESERVED}, R.E_PARA), ({"alg": 77}, R.E_PARA),
                         ({"low": 5}, R.E_PARA), ({"i": [i[0] + 64] + i[1:]}, R.E_PARA),
                         ({"i": [0] + i[1:]}, R.E_PTR), ({"dt": DT.INT16, "op": OP.PROD}, R.E_PARA),
                         ({"i": i * 9, "o": o * 9}, R.E_PARA)):
        with pytest.raises(h.HcommError) as e:
            mk(**kwargs)
        assert e.value.code == code, kwargs
    with pytest.raises(h.HcommError) as e:                      # the reference refuses bf16 PROD as well as int16
        mk(dt=DT.BFP16, op=OP.PROD)
    assert e.value.code == R.E_PARA
    mk(dt=DT.FP16, op=OP.PROD).destroy()
    p = mk(alg=h.Alg.ALLREDUCE_RHD, low=h.Lowering.FUSED)
    assert [r.kind for r in p.launches()] == [h.Kernel.TREE]
    p.destroy()


def test_fused_deterministic_reduce_scatter_is_one_tree_launch_with_the_hand_derived_trees():
    """Leaf position q of destination d holds rank d - bitrev(q) where bitrev(q) < n; level l folds position
    q + 2^l into q.  That tree must be the hand-derived one of the step-wise schedule (tail fold, then halving)."""
    import json
    import os
    gold = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "schedules_hand_derived.json")))
    for n_s, trees in gold["rs_local_reduce_rank_tree"].items():
        if n_s.startswith("_"):
            continue
        n = int(n_s)
        L = max(1, (n - 1).bit_length())
        K = 1 << L
        rev = lambda q: int(format(q, "0%db" % L)[::-1], 2)
        for d_s, tree in trees.items():
            x = [(int(d_s) - rev(q)) % n if rev(q) < n else None for q in range(K)]
            for l in range(L):
                for q in range(0, K, 2 << l):
                    if x[q + (1 << l)] is not None:
                        x[q] = [x[q], x[q + (1 << l)]]
            assert x[0] == tree, (n, d_s)
    for n in (2, 3, 5, 8, 17, 32):
        i, o = ptrs(n, 1 << 24)
        p = h.Plan(h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, h.Lowering.FUSED, i, o, 4096, DT.BFP16, OP.SUM)  # no scratch
        recs = p.launches()
        assert [r.kind for r in recs] == [h.Kernel.TREE] and recs[0].nseg == n and recs[0].bytes == n * 8192
        assert p.info.movedBytes == (n + 1) * n * 8192
        stepwise_scratch = h.scratch_bytes(h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, n, 4096, DT.BFP16)
        assert stepwise_scratch > 0
        p.destroy()
        with pytest.raises(h.HcommError) as e:      # slices that are not 16-byte multiples
            h.Plan(h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, h.Lowering.FUSED, i, o, 4099, DT.BFP16, OP.SUM)
        assert e.value.code == R.E_NOT_SUPPORT
        with pytest.raises(h.HcommError) as e:      # the step-wise replay still needs its communication buffers
            h.Plan(h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, h.Lowering.STEPWISE, i, o, 4096, DT.BFP16, OP.SUM)
        assert e.value.code == R.E_PTR


def test_fused_chunk_mesh_is_chain_launches_over_whole_ranks_sub_chunks():
    for n, count, launches, nseg in ((2, 1 << 20, 1, [2]), (6, 1 << 20, 1, [30]), (8, 1 << 20, 2, [28, 28]),
                                     (17, 1 << 22, 9, [32] * 8 + [16]), (32, 1 << 22, 32, [31] * 32), (8, 100, 1, [4])):
        i, o = ptrs(n, 1 << 26)
        p = h.Plan(h.Alg.ALLREDUCE_CHUNK_MESH, h.Lowering.FUSED, i, o, count, DT.FP32, OP.SUM)   # no scratch buffers
        recs = p.launches()
        assert [r.kind for r in recs] == [h.Kernel.CHAIN] * launches, n
        assert [r.nseg for r in recs] == nseg, n
        assert sum(r.bytes for r in recs) == 4 * count                 # every element of the message folded once
        assert p.info.movedBytes == 2 * n * 4 * count                  # n reads and n writes per element
        q = h.Plan(h.Alg.ALLREDUCE_CHUNK_MESH, h.Lowering.STEPWISE, i, o, count, DT.FP32, OP.SUM, 0, ptrs(n, 1 << 26)[0])
        assert p.info.algorithmicBytes == q.info.algorithmicBytes
        p.destroy()
        q.destroy()


def test_keep_inputs_lowering_moves_one_read_per_input_and_one_write_per_output():
    for alg, n, count, moved in ((h.Alg.ALLREDUCE_RING, 8, 1 << 20, 16), (h.Alg.ALLREDUCE_RHD, 16, 1 << 20, 32),
                                 (h.Alg.ALLREDUCE_RHD, 6, 1 << 20, 12), (h.Alg.ALLREDUCE_NHR, 7, 7 << 18, 14),
                                 (h.Alg.ALLREDUCE_NB, 5, 5 << 18, 10), (h.Alg.ALLREDUCE_MESH_ONESHOT, 8, 1 << 20, 72),
                                 (h.Alg.ALLREDUCE_NHR_ONESHOT, 8, 1 << 20, 16), (h.Alg.ALLREDUCE_LOCAL_REDUCE, 8, 1 << 20, 16)):
        i, o = ptrs(n, 1 << 24)
        p = h.Plan(alg, h.Lowering.FUSED_KEEP_INPUTS, i, o, count, DT.FP32, OP.SUM)
        q = h.Plan(alg, h.Lowering.FUSED, i, o, count, DT.FP32, OP.SUM)
        assert p.info.movedBytes == moved * count * 4, alg             # (reads + writes) x message bytes
        assert p.info.movedBytes <= q.info.movedBytes and p.info.algorithmicBytes == q.info.algorithmicBytes
        assert [(r.kind, r.nseg, r.bytes) for r in p.launches()] == [(r.kind, r.nseg, r.bytes) for r in q.launches()]
        p.destroy()
        q.destroy()
    i, o = ptrs(4, 1 << 20)
    with pytest.raises(h.HcommError) as e:          # the in-place stage's result lives in the input
        h.Plan(h.Alg.REDUCE_SCATTER_RING, h.Lowering.FUSED_KEEP_INPUTS, i, None, 4096, DT.FP32, OP.SUM)
    assert e.value.code == R.E_NOT_SUPPORT
    with pytest.raises(h.HcommError) as e:
        h.Plan(h.Alg.ALLREDUCE_RING, 3, i, o, 4096, DT.FP32, OP.SUM)
    assert e.value.code == R.E_PARA


def test_counts_whose_byte_offsets_would_leave_64_bits_are_refused():
    i, o = ptrs(4, 4096)
    for count in (2**48 + 1, 2**62, 2**64 - 1):
        for low in (h.Lowering.STEPWISE, h.Lowering.FUSED):
            with pytest.raises(h.HcommError) as e:
                h.Plan(h.Alg.ALLREDUCE_RING, low, i, o, count, DT.FP32, OP.SUM)
            assert e.value.code == R.E_PARA
        with pytest.raises(h.HcommError) as e:
            h.schedule_emit(h.Alg.REDUCE_SCATTER_MESH, 4, 16, DT.INT8, stride=count)
        assert e.value.code == R.E_PARA
        with pytest.raises(h.HcommError) as e:
            h.scratch_bytes(h.Alg.ALLREDUCE_CHUNK_MESH, 4, count, DT.INT32)
        assert e.value.code == R.E_PARA
    with pytest.raises(h.HcommError) as e:
        h.calc_slices(2**61, 4, 8)
    assert e.value.code == R.E_PARA
    assert sum(sz for _, sz in h.calc_slices(2**60, 4, 8)) == 2**62


@pytest.mark.parametrize("name,alg,n,count,dt,launches,algo_bytes,moved_fused", [
    # the five benchmark configurations at full size: launch structure and byte accounting, no memory touched
    ("cfg1", h.Alg.ALLREDUCE_RING, 8, 1048576, DT.FP32, 15, 155189248, 23 * 4194304),
    ("cfg2", h.Alg.ALLREDUCE_RING, 8, 67108864, DT.BFP16, 15, 4966055936, 23 * 134217728),
    ("cfg3", h.Alg.ALLREDUCE_RHD, 16, 33554432, DT.INT32, 10, 10334765056, 40 * 134217728),  # last gather: 2 x 512 MiB
    ("cfg4", h.Alg.ALLREDUCE_MESH_ONESHOT, 8, 2097152, DT.FP16, 8, 8 * 23 * 4194304, 72 * 4194304),
    ("cfg5a", h.Alg.REDUCE_SCATTER_RING, 7, 100000003, DT.FP32, 16, 7200000216, 13 * 400000012),  # 3 pieces x 6 steps
    ("cfg5b", h.Alg.REDUCE_SCATTER_RING, 7, 100000003, DT.INT8, 6, 1800000054, 13 * 100000003),
])
def test_plan_structure_of_benchmark_configs(rec, name, alg, n, count, dt, launches, algo_bytes, moved_fused):
    size = count * h.DTYPE_SIZE[dt]
    i, o = ptrs(n, size)
    op = OP.PROD if name == "cfg5a" else OP.SUM
    p = h.Plan(alg, h.Lowering.STEPWISE, i, o, count, dt, op)
    assert (p.info.launches, p.info.algorithmicBytes, p.info.movedBytes) == (launches, algo_bytes, algo_bytes)
    # one launch = one step of all ranks; a copy step that writes more than 512 MiB is cut in two; steps that write
    # more than 2.5 times what the memory-side cache serves well (cfg5a: 400 MB) run piece by piece, and the last step of
    # a piece shares its launch with the first step of the next, which touches other memory
    assert all(r.nseg == n or (r.kind == h.Kernel.COPY and r.bytes == 512 << 20) or (name == "cfg5a" and r.nseg == 2 * n)
               for r in p.launches())
    if name == "cfg5a":
        assert [r.nseg for r in p.launches()] == [7] * 5 + [14] + [7] * 4 + [14] + [7] * 5
        assert all(r.bytes <= 2 * (128 << 20) for r in p.launches())
    h.HcommGfxLaunchLogClear(rec)
    assert p.run(rec) == 0
    assert [(r.kind, r.nseg, r.bytes) for r in h.launch_log(rec)] == [(r.kind, r.nseg, r.bytes) for r in p.launches()]
    p.destroy()
    if moved_fused is not None:
        p = h.Plan(alg, h.Lowering.FUSED, i, o, count, dt, op)
        assert (p.info.launches, p.info.algorithmicBytes, p.info.movedBytes) == (1, algo_bytes, moved_fused)
        assert [r.kind for r in p.launches()] == [h.Kernel.TREE if alg == h.Alg.ALLREDUCE_RHD else h.Kernel.CHAIN]
        p.destroy()


def test_fused_rhd_byte_accounting_with_fold():
    """6 ranks: block of 4, block ranks 0 and 1 (ranks 0, 2) absorb ranks 1, 3.  Per element: 4 leaf reads + 2
    neighbour reads + 2 stores on even positions + 6 outputs = 14 transfers, + 1 for each absorbing block rank
    that sits on an odd position for the slice (block rank b is odd-positioned for slice c iff (b^c) & 2):
    slices 0, 1 -> none; slices 2, 3 -> both."""
    i, o = ptrs(6, 4096)
    p = h.Plan(h.Alg.ALLREDUCE_RHD, h.Lowering.FUSED, i, o, 1024, DT.FP32, OP.SUM)
    assert p.info.movedBytes == 2 * 1024 * 14 + 2 * 1024 * 16
    p.destroy()


def test_plan_from_a_callers_op_list(rec):
    """A caller's own op list lowers exactly like the built-in schedule it was taken from; malformed lists are refused."""
    n, count, dt = 5, 4099, DT.FP32
    ins = [DST + (i << 22) for i in range(n)]
    outs = [SRC + (i << 22) for i in range(n)]
    ops = h.schedule_emit(h.Alg.ALLREDUCE_NHR, n, count, dt)
    mine = h.OpListPlan(ops, n, {0: ins, 1: outs}, dt, OP.SUM)
    ref = h.Plan(h.Alg.ALLREDUCE_NHR, h.Lowering.STEPWISE, ins, outs, count, dt, OP.SUM)
    assert [(l.kind, l.nseg, l.bytes, l.blocks) for l in mine.launches()] == \
        [(l.kind, l.nseg, l.bytes, l.blocks) for l in ref.launches()]
    assert (mine.info.steps, mine.info.algorithmicBytes) == (ref.info.steps, ref.info.algorithmicBytes)
    assert mine.run(rec) == 0
    for bad, code in ((ops[::-1], R.E_PARA),                                        # not ordered by step
                      ([(0, 1, 0, 0, 0, 1, 0, 0, 6)], R.E_PARA),                     # a reduce of 1.5 elements
                      ([(0, 2, 0, 0, 0, 1, 0, 0, 8)], R.E_PARA),                     # unknown kind
                      ([(0, 0, 7, 0, 0, 1, 0, 0, 8)], R.E_PARA),                     # rank out of range
                      ([(0, 0, 0, 5, 0, 1, 0, 0, 8)], R.E_PARA),                     # buffer role out of range
                      ([(0, 0, 0, 2, 0, 1, 0, 0, 8)], R.E_PTR)):                     # role without buffers
        with pytest.raises(h.HcommError) as e:
            h.OpListPlan(bad, n, {0: ins, 1: outs}, dt, OP.SUM)
        assert e.value.code == code
    empty = h.OpListPlan([], n, {0: ins}, dt, OP.SUM)
    assert empty.info.launches == 0 and empty.run(rec) == 0


def test_steps_that_mix_reduces_and_copies_lower_to_one_launch_per_kind(rec):
    """The double-ring reduce-scatter pairs every reduce with the fetch of the next slice from the user input: a step
    of 8 ranks x 2 rings is one reduce launch and one copy launch, not 32 alternating ones.  A step whose operations
    could observe each other keeps its order."""
    n, count, dt = 8, 1 << 20, DT.FP32
    bufs = [[DST + (role << 34) + (i << 26) for i in range(n)] for role in range(4)]
    p = h.DoubleRingPlan(h.Alg.ALLREDUCE_RING, 1, n, bufs[0], bufs[1], bufs[2], bufs[3], 8 << 20, count, dt, OP.SUM)
    kinds = [l.kind for l in p.launches()]
    K = h.Kernel
    assert kinds == [K.COPY] + [K.REDUCE2, K.COPY] * (n - 2) + [K.REDUCE2] + [K.COPY] + [K.COPY] * (n - 1)
    assert [l.nseg for l in p.launches()][:3] == [32, 16, 16]
    assert p.run(rec) == 0
    p.destroy()
    # copy A -> B, then B += C, then copy B -> D, all in one step: each reads what the one before wrote
    A, B, C_, D = (DST + (i << 22) for i in range(4))
    ops = [(0, 0, 0, 0, 1 << 22, 0, 0, 0, 4096), (0, 1, 0, 0, 1 << 22, 0, 0, 2 << 22, 4096),
           (0, 0, 0, 0, 3 << 22, 0, 0, 1 << 22, 4096)]
    q = h.OpListPlan(ops, 1, {0: [DST]}, dt, OP.SUM)
    assert [l.kind for l in q.launches()] == [K.COPY, K.REDUCE2, K.COPY]
    q.destroy()


def test_plan_run_checks(rec):
    i, o = ptrs(2, 4096)
    p = h.Plan(h.Alg.ALLREDUCE_RING, h.Lowering.STEPWISE, i, o, 1024, DT.FP32, OP.SUM)
    assert p.run(0) == R.E_PTR
    assert p.run_range(rec, 0, p.info.launches + 1) == R.E_PARA
    assert p.run_range(rec, p.info.launches, 0) == R.SUCCESS
    assert raw._plan_run(None, rec) == R.E_PTR
    p.destroy()


def test_thread_alloc_without_gpu_is_unavailable():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    code, _ = h.HcommThreadAlloc(h.CommEngine.CPU_TS, 1, 0)
    assert code == R.E_UNAVAIL                                      # fails loudly, no CPU fallback
    code, _ = h.HcommThreadAllocWithStream(0, 0)
    assert code == R.E_UNAVAIL


# ---- the entry point for callers that cannot allocate ----------------------------------------------------------

def _launch_tuples(records):
    return [(r.kind, r.dtype, r.op, r.nseg, r.bytes, r.blocks) for r in records]


@pytest.mark.parametrize("n,count,dt", [(8, 1048576 + 37, DT.BFP16), (4, 500001, DT.FP32), (2, 3, DT.FP16), (1, 77, DT.INT8)])
def test_no_alloc_allreduce_submits_the_plans_launches(rec, n, count, dt):
    """HcommGfxAllReduceLocalReduceNoAlloc submits exactly the launches of the step-wise plan that is given
    communication buffers (same kinds, segments, bytes and grids), in the same order."""
    ins = [0x1000000 * (r + 1) for r in range(n)]
    outs = [(1 << 36) + 0x1000000 * (r + 1) for r in range(n)]
    sb = h.scratch_bytes(h.Alg.ALLREDUCE_LOCAL_REDUCE, n, count, dt)
    scr = [(1 << 38) + ((sb + 255) // 256 * 256) * r for r in range(n)] if sb else None
    plan = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.STEPWISE, ins, outs, count, dt, OP.SUM, 0, scr)
    want = _launch_tuples(plan.launches())
    plan.destroy()
    h.HcommGfxLaunchLogClear(rec)
    assert h.HcommGfxAllReduceLocalReduceNoAlloc(rec, ins, outs, count, dt, OP.SUM) == R.SUCCESS
    assert _launch_tuples(h.launch_log(rec)) == want


def test_no_alloc_allreduce_checks(rec):
    f = h.HcommGfxAllReduceLocalReduceNoAlloc
    ins = [0x1000000 * (r + 1) for r in range(16)]
    outs = [(1 << 36) + 0x1000000 * (r + 1) for r in range(16)]
    assert f(rec, ins[:8], outs[:8], 1 << 20, DT.BFP16, OP.SUM) == R.SUCCESS
    assert f(0, ins[:8], outs[:8], 16, DT.BFP16, OP.SUM) == R.E_PTR                       # no thread
    assert f(rec, ins[:3] + [None], outs[:4], 16, DT.BFP16, OP.SUM) == R.E_PTR              # a rank without a buffer
    assert f(rec, ins[:3] + [ins[3] + 64], outs[:4], 16, DT.BFP16, OP.SUM) == R.E_PARA      # not on 128 bytes
    assert f(rec, ins[:16], outs[:16], 16, DT.BFP16, OP.SUM) == R.E_PARA                    # more ranks than it takes
    assert f(rec, ins[:8], outs[:8], 16, DT.BFP16, OP.PROD) == R.E_PARA                     # bf16 has no PROD
    assert f(rec, ins[:8], outs[:8], 16, DT.INT64, OP.SUM) == R.E_PARA
    # the communication buffers of 8 ranks must fit the library's array: 8 MiB each
    per_rank = h.NOALLOC_SCRATCH_BYTES // 8
    fits = per_rank // 2 - 8 * 16384  # bf16 elements; slots are rounded up to 16 KiB
    assert h.scratch_bytes(h.Alg.ALLREDUCE_LOCAL_REDUCE, 8, fits, DT.BFP16) <= per_rank
    assert f(rec, ins[:8], outs[:8], fits, DT.BFP16, OP.SUM) == R.SUCCESS
    h.HcommGfxLaunchLogClear(rec)
    assert f(rec, ins[:8], outs[:8], per_rank // 2 + 1, DT.BFP16, OP.SUM) == R.E_PARA
    assert h.launch_log(rec) == []                                                          # refused before any launch
    # the rank counts the algorithm itself refuses stay refused
    code3 = f(rec, ins[:3], outs[:3], 100, DT.BFP16, OP.SUM)
    try:
        h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.STEPWISE, ins[:3], outs[:3], 100, DT.BFP16, OP.SUM, 0,
               [(1 << 38) + 0x100000 * r for r in range(3)]).destroy()
        plan_code = R.SUCCESS
    except h.HcommError as e:
        plan_code = e.code
    assert code3 == plan_code


def test_direct_launch_switch_returns_the_previous_setting():
    before = h.HcommGfxSetDirectLaunches(0)
    try:
        assert h.HcommGfxSetDirectLaunches(1) == 0
        assert h.HcommGfxSetDirectLaunches(5) == 1   # any non-zero value means on
        assert h.HcommGfxSetDirectLaunches(0) == 1
    finally:
        h.HcommGfxSetDirectLaunches(before)
    assert h.HcommGfxSetDirectLaunches(before) == before


def test_launch_records_name_the_grid_shape():
    """rows / streaming of HcommGfxLaunchRecord: which kernel variant a launch takes, decided on the host."""
    K = h.Kernel
    # 8-rank ring allreduce, 128 MiB per rank: every step is 8 slices of 16 MiB = 1024 tiles each -> a grid of
    # 1024 x 8; the reduces (128 MiB written, more than 64) take the streaming shape, the copies (less than 256) the other
    size = 128 << 20
    i, o = ptrs(8, size, base=1 << 40)
    p = h.Plan(h.Alg.ALLREDUCE_RING, h.Lowering.STEPWISE, i, o, size // 2, DT.BFP16, OP.SUM)
    recs = p.launches()
    assert len(recs) == 15
    assert all(r.rows == 1024 and r.streaming == (r.kind == K.REDUCE2) and r.blocks == 8 * 1024 for r in recs)
    p.destroy()
    # 16-rank recursive halving-doubling: the first halving step writes 16 x 64 MiB = 1 GiB -> streaming, 4096 tiles a row
    i, o = ptrs(16, size, base=1 << 40)
    p = h.Plan(h.Alg.ALLREDUCE_RHD, h.Lowering.STEPWISE, i, o, size // 4, DT.INT32, OP.SUM)
    first = [r for r in p.launches() if r.kind == K.REDUCE2][0]
    assert (first.rows, first.streaming, first.nseg) == (4096, 1, 16)
    p.destroy()
    # small fused launches: addresses resolved on the host
    i, o = ptrs(8, 4096, base=1 << 40)
    for alg, kind in ((h.Alg.ALLREDUCE_MESH_ONESHOT, K.CHAIN), (h.Alg.ALLREDUCE_RING, K.CHAIN), (h.Alg.ALLREDUCE_NHR, K.TREE)):
        p = h.Plan(alg, h.Lowering.FUSED, i, o, 2048, DT.FP16, OP.SUM)
        assert [(r.kind, r.rows) for r in p.launches()] == [(kind, 1)]
        p.destroy()
    # recursive halving on 6 ranks absorbs the odd neighbours before the tree: not a launch the host can resolve
    i, o = ptrs(6, 6 * 4096, base=1 << 40)
    p = h.Plan(h.Alg.ALLREDUCE_RHD, h.Lowering.FUSED, i, o, 6 * 1024, DT.FP32, OP.SUM)
    assert [(r.kind, r.rows) for r in p.launches()] == [(K.TREE, 0)]
    p.destroy()
    # segments of very different lengths beyond the small-launch limit keep the one-dimensional grid
    code, rec = h.HcommGfxRecorderThreadAlloc()
    assert code == 0
    h.check(h.HcommBatchModeStart(b"ragged"), "start")
    base = 1 << 40
    for k, n in enumerate((16 << 20, 16 << 10, 32 << 20, 4096)):
        h.check(h.HcommLocalCopyOnThread(rec, base + (2 * k) * (64 << 20), base + (2 * k + 1) * (64 << 20), n), "copy")
    h.check(h.HcommBatchModeEnd(b"ragged"), "end")
    log = h.launch_log(rec)
    assert [(r.kind, r.nseg, r.rows) for r in log] == [(K.COPY, 4, 0)]
    h.HcommThreadFree([rec])
    # with the switch off nothing takes a two-dimensional grid
    before = h.HcommGfxSetDirectLaunches(0)
    try:
        i, o = ptrs(8, 4096, base=1 << 40)
        for low in (h.Lowering.STEPWISE, h.Lowering.FUSED):
            p = h.Plan(h.Alg.ALLREDUCE_RING, low, i, o, 1024, DT.FP32, OP.SUM)
            assert all(r.rows == 0 for r in p.launches())
            p.destroy()
    finally:
        h.HcommGfxSetDirectLaunches(before)


# ---- the NIC-plugin face of the library ---------------------------------------------------------------------------

def test_nic_plugin_tables_have_the_references_layout_and_refuse_what_needs_a_network(rec):
    """hcomm_nic_plugin.h:23-104 as the reference's plugin manager checks it (nic_plugin_manager.cc:61-79,206-270):
    magic words, versions, sizes, one protocol from the plugins' own range; the data-plane entries run on a thread of
    this library (a recorder here: launches are logged), everything that needs a network says HCCL_E_NOT_SUPPORT."""
    from hcomm_amd import nic_plugin as P
    info = P.get_info()
    assert (info.header.version, info.header.magicWord, info.header.size) == (1, 0x0fcf0f1f, 112)
    assert info.name == b"hcomm_gfx" and info.protocolCount == 1 and info.protocols[0] >= 1000
    assert C.sizeof(P.CommAbiHeader) == 16 and C.sizeof(P.ChannelOps) == 208 and C.sizeof(P.EndpointOps) == 80
    assert C.sizeof(P.PluginInfo) == 112 and C.sizeof(P.CommMem) == 24
    assert P.create_endpoint(None)[0] == R.E_PTR
    code, ep_ctx, ep = P.create_endpoint(P.endpoint_desc())
    assert code == R.SUCCESS
    assert (ep.header.version, ep.header.magicWord, ep.header.size) == (1, 0x0fcf0f2f, 80)
    assert ep.init(ep_ctx) == R.SUCCESS
    assert ep.getListenPort(ep_ctx, None) == R.E_NOT_SUPPORT
    assert ep.registerMemory(ep_ctx, None, None, None) == R.E_NOT_SUPPORT
    assert P.create_channel(None, P.channel_desc(3))[0] == R.E_PTR
    assert P.create_channel(ep_ctx, None)[0] == R.E_PTR
    code, ch_ctx, ch = P.create_channel(ep_ctx, P.channel_desc(3))
    assert code == R.SUCCESS
    assert (ch.header.version, ch.header.magicWord, ch.header.size) == (1, 0x0fcf0f3f, 208)
    assert ch.init(ch_ctx) == R.SUCCESS
    status = C.c_int32(-1)
    assert ch.getStatus(ch_ctx, C.byref(status)) == R.SUCCESS and status.value == 0
    # data plane on a thread: the same checks, in the same order, as the primitives
    h.HcommGfxLaunchLogClear(rec)
    assert ch.writeReduceOnThread(ch_ctx, rec, None, SRC, 4, DT.FP32, OP.SUM) == R.E_PTR
    assert ch.writeReduceOnThread(ch_ctx, rec, DST, SRC, 4, DT.INT64, OP.SUM) == R.E_PARA
    assert ch.writeReduceOnThread(ch_ctx, 0, DST, SRC, 4, DT.FP32, OP.SUM) == R.E_PTR
    assert ch.writeReduceOnThread(None, rec, DST, SRC, 4, DT.FP32, OP.SUM) == R.E_PTR
    assert ch.writeReduceOnThread(ch_ctx, rec, DST, SRC, 1 << 20, DT.BFP16, OP.MAX) == R.SUCCESS
    assert ch.readReduceOnThread(ch_ctx, rec, DST, SRC, 1 << 20, DT.BFP16, OP.MAX) == R.SUCCESS
    assert ch.writeOnThread(ch_ctx, rec, DST, SRC, 4096) == R.SUCCESS
    assert ch.readNbiOnThread(ch_ctx, rec, DST, SRC, 4096) == R.SUCCESS
    descs = (h.BatchTransferDesc * 2)(h.desc_reduce(DST, SRC, 256, DT.FP32, OP.SUM),
                                      h.desc_reduce(DST + (1 << 24), SRC + (1 << 24), 256, DT.FP32, OP.SUM, read=True))
    assert ch.batchTransferOnThread(ch_ctx, rec, descs, 2) == R.SUCCESS
    log = h.launch_log(rec)
    assert [(r.kind, r.nseg) for r in log] == [(h.Kernel.REDUCE2, 1), (h.Kernel.REDUCE2, 1), (h.Kernel.COPY, 1),
                                               (h.Kernel.COPY, 1), (h.Kernel.REDUCE2, 2)]
    # what needs a host-side engine or a remote process
    assert ch.writeNbi(ch_ctx, DST, SRC, 16) == R.E_NOT_SUPPORT
    assert ch.readNbi(ch_ctx, DST, SRC, 16) == R.E_NOT_SUPPORT
    assert ch.writeWithNotifyOnThread(ch_ctx, rec, DST, SRC, 16, 0) == R.E_NOT_SUPPORT
    assert ch.writeReduceWithNotifyOnThread(ch_ctx, rec, DST, SRC, 4, DT.FP32, OP.SUM, 0) == R.E_NOT_SUPPORT
    assert ch.notifyRecord(ch_ctx, 0) == R.E_NOT_SUPPORT and ch.notifyWait(ch_ctx, 0, 1) == R.E_NOT_SUPPORT
    # the channel's own notifies: three of them, each record consumed by one wait
    assert ch.notifyWaitOnThread(ch_ctx, rec, 0, 1) == R.E_TIMEOUT
    assert ch.notifyRecordOnThread(ch_ctx, rec, 3) == R.E_PARA
    assert ch.notifyRecordOnThread(ch_ctx, rec, 2) == R.SUCCESS
    assert ch.notifyWaitOnThread(ch_ctx, rec, 1, 1) == R.E_TIMEOUT
    assert ch.notifyWaitOnThreadWithDefaultTimeout(ch_ctx, rec, 2) == R.SUCCESS
    assert ch.notifyWaitOnThread(ch_ctx, rec, 2, 1) == R.E_TIMEOUT
    assert ch.fence(ch_ctx) == R.SUCCESS and ch.fenceOnThread(ch_ctx, rec) == R.SUCCESS
    assert ch.drainOnThread(ch_ctx, rec) == R.SUCCESS and ch.drainOnThread(ch_ctx, 12345) == R.E_PTR
    assert ch.destroy(ch_ctx) == R.SUCCESS
    assert ep.destroy(ep_ctx) == R.SUCCESS


def test_direction_of_large_launches_follows_what_they_read(rec):
    """A copy / two-input reduce launch that writes more than HcommGfxSetAlternateBytes and reads what one of the thread's
    last two such launches wrote walks the other way than that launch did; one that reads nothing of theirs walks
    forwards; smaller launches and folds are left alone.  (Recorder thread: the decision is host logic.)"""
    n, count, dt = 8, 1 << 26, h.HcommDataType.BFP16          # 8 x 128 MiB: every ring step writes exactly 128 MiB
    i, o = _fake(n, 1 << 40), _fake(n, 1 << 41)
    plan = h.Plan(h.Alg.ALLREDUCE_RING, h.Lowering.STEPWISE, i, o, count, dt, 0)
    h.HcommGfxLaunchLogClear(rec)
    assert plan.run(rec) == 0
    assert [l.backwards for l in h.launch_log(rec)] == [0] * 15                 # 128 MiB is not MORE than 128 MiB
    before = h.HcommGfxSetAlternateBytes(1 << 20)
    try:
        assert before == 128 << 20
        h.HcommGfxLaunchLogClear(rec)
        assert plan.run(rec) == 0
        # every step reads what the step before wrote - also the first gather copy, which reads the last fold's result
        assert [l.backwards for l in h.launch_log(rec)] == [s % 2 for s in range(15)]
        # a fetch of fresh data between two folds walks forwards, and the fold after it against the LATER writer
        A, B, C_, D, U = (x << 40 for x in (3, 4, 5, 6, 7))
        h.HcommGfxLaunchLogClear(rec)
        nbytes = 4 << 20
        assert h.HcommLocalCopyOnThread(rec, A, U, nbytes) == 0                               # reads nothing recent: forwards
        assert h.HcommLocalReduceOnThread(rec, B, A, nbytes // 2, dt, 0) == 0                 # reads A: backwards
        assert h.HcommLocalCopyOnThread(rec, C_, U + nbytes, nbytes) == 0                     # fresh: forwards
        assert h.HcommLocalReduceOnThread(rec, B, C_, nbytes // 2, dt, 0) == 0                # reads C (forwards) and B (backwards): the later one decides
        assert h.HcommLocalReduceOnThread(rec, D, A, nbytes // 2, dt, 0) == 0                 # A was written three launches ago: forgotten, forwards
        assert h.HcommLocalCopyOnThread(rec, A, D, 4096) == 0                                 # small: left alone
        assert [l.backwards for l in h.launch_log(rec)] == [0, 1, 0, 1, 0, 0]
        assert h.HcommGfxSetAlternateBytes(0) == 1 << 20                                      # never
        h.HcommGfxLaunchLogClear(rec)
        assert plan.run(rec) == 0
        assert [l.backwards for l in h.launch_log(rec)] == [0] * 15
        assert h.HcommGfxSetAlternateBytes(1 << 20) == 0
    finally:
        h.HcommGfxSetAlternateBytes(before)
    plan.destroy()


def test_steps_larger_than_the_cache_run_piece_by_piece(rec):
    """A step-wise plan whose steps write more than 320 MiB, made of operations that are whole slices (any two ranges
    the same or apart), is lowered piece by piece: all steps on the first part of every slice, then all steps on the
    second, ... each launch writing about 128 MiB, no piece shorter than 16 MiB.  Schedules with nested ranges
    (halving-doubling), short slices or smaller steps keep one launch per step; HCOMM_GFX_PIECE_BYTES=0 (a process of
    its own: read once) keeps every plan that way."""
    import subprocess
    import sys
    key = lambda p: [(l.kind, l.nseg, l.bytes) for l in p.launches()]
    i, o = _fake(8, 1 << 40), _fake(8, 1 << 41)
    big = [x * 64 for x in i], [x * 64 for x in o]                      # 4 GiB apart
    p = h.Plan(h.Alg.ALLREDUCE_RING, h.Lowering.STEPWISE, big[0], big[1], 1 << 28, h.HcommDataType.BFP16, 0)   # 8 x 512 MiB
    assert p.info.launches == 4 * 15 and set(l.bytes for l in p.launches()) == {128 << 20}
    assert [l.kind for l in p.launches()] == ([1] * 7 + [0] * 8) * 4
    assert p.info.algorithmicBytes == (3 * 7 + 2 * 8) * (64 << 20) * 8
    p.destroy()
    p = h.Plan(h.Alg.ALLREDUCE_RING, h.Lowering.STEPWISE, big[0], big[1], 1 << 27, h.HcommDataType.BFP16, 0)   # steps of 256 MiB: as they are
    assert p.info.launches == 15
    p.destroy()
    i16, o16 = [(1 << 40) + r * (1 << 32) for r in range(16)], [(1 << 44) + r * (1 << 32) for r in range(16)]
    p = h.Plan(h.Alg.ALLREDUCE_RHD, h.Lowering.STEPWISE, i16, o16, 1 << 25, h.HcommDataType.INT32, 0)            # nested ranges
    assert p.info.launches == 10
    p.destroy()
    scr = [(1 << 52) + r * (1 << 32) for r in range(8)]
    p = h.Plan(h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, h.Lowering.STEPWISE, big[0], big[1], 1 << 23, h.HcommDataType.BFP16, 0,
               scratch_ptrs=scr)                                                                                   # 1 GiB steps of 16 MiB slices: too short to cut
    assert p.info.launches == 5
    p.destroy()
    child = ("import sys; sys.path.insert(0, %r); import hcomm_amd as h\n"
             "i=[(1<<46)+r*(1<<34) for r in range(8)]; o=[(1<<50)+r*(1<<34) for r in range(8)]\n"
             "p=h.Plan(h.Alg.ALLREDUCE_RING,h.Lowering.STEPWISE,i,o,1<<28,h.HcommDataType.BFP16,0); print(p.info.launches)") % ROOT
    run = subprocess.run([sys.executable, "-c", child], capture_output=True, text=True, env=dict(os.environ, HCOMM_GFX_PIECE_BYTES="0"))
    assert run.stdout.split() == ["15"], (run.stdout, run.stderr[-500:])


def test_a_whole_collective_in_one_batch_is_cut_into_the_plans_pieces():
    """Benchmark configuration 5a (7 ranks x 100,000,003 fp32, steps of 400 MB) given as a thread per rank with posts
    and waits inside one batch: HcommBatchModeEnd's rounds are the schedule's steps, so it cuts them into the same
    three pieces as the step-wise plan and issues the plan's sixteen launches."""
    from hcomm_amd import caller
    n, count, dt = 7, 100000003, h.HcommDataType.FP32
    recs = [h.HcommGfxRecorderThreadAlloc()[1] for _ in range(n)]
    try:
        i = [(1 << 40) + r * (1 << 32) for r in range(n)]
        o = [(1 << 44) + r * (1 << 32) for r in range(n)]
        rp = caller.Replay(h.schedule_emit(h.Alg.REDUCE_SCATTER_RING, n, count, dt), {0: i, 1: o}, dt, 0)
        code, st = rp.run_on_threads_batched(recs)
        assert code == 0
        plan = h.Plan(h.Alg.REDUCE_SCATTER_RING, h.Lowering.STEPWISE, i, o, count, dt, 0)
        key = lambda l: (l.kind, l.nseg, l.bytes, l.dtype, l.op)
        assert [key(l) for l in h.launch_log(recs[0])] == [key(l) for l in plan.launches()]
        assert plan.info.launches == 16
        # the same without notifies: every call on ONE thread between one Start / End pair - the steps are told
        # apart by what they touch
        h.HcommGfxLaunchLogClear(recs[1])
        code, st = rp.run_one_batch(recs[1])
        assert code == 0 and st.batches == 1
        assert [key(l) for l in h.launch_log(recs[1])] == [key(l) for l in plan.launches()]
        # and a batch per step stays a launch per step: one step alone has nobody to find its pieces cached
        h.HcommGfxLaunchLogClear(recs[2])
        code, st = rp.run_batched(recs[2])
        assert code == 0 and len(h.launch_log(recs[2])) == 6
        plan.destroy()
    finally:
        h.HcommThreadFree(recs)
