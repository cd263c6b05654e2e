"""Whole schedules through the reference's own boundary, the way its caller drives it (hcomm_amd/csrc/hg_caller.c binds
the library with dlsym and uses nothing but HcommBatchModeStart / End, HcommLocalCopyOnThread, HcommLocalReduceOnThread
and the thread notifies):
  batched     one Start / End pair per schedule step on one thread (cpu_primitives_c_adpt.cc:58-130,
              launch_context.cc:139-174);
  per rank    rank r's calls on thread r, eagerly, each thread posting to and waiting for the peers it exchanges data
              with between the steps (reduce_scatter_ring.cc:211-217,254-272) - issued by one host thread for all
              ranks, or by a host thread per rank (the ranks of the reference are processes of their own), where a wait
              may reach the library before its record and sits on the host until the record has been issued;
  one batch   the per-rank calls, posts and waits included, between ONE Start / End pair: the collective as one batch
              over all its threads (launch_context.cc:16-44), which HcommBatchModeEnd turns into the launches of the
              step-wise plan.
Every one of the 2N rank buffers (and the communication buffers, where a schedule has them) is compared bit for bit
with the CPU oracle's replay."""
import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import caller
from util import DT, OPS, assert_same, from_dev, gen, to_dev
from test_gpu_collectives import ALGS, buffer_counts, say

pytestmark = pytest.mark.gpu

CASES = [
    # alg, n, count, dtype, op
    ("ring_ar", 8, 1 << 20, "fp32", "sum"),         # benchmark config 1
    ("ring_ar", 8, 1000003, "bf16", "sum"),         # benchmark config 2, scaled down, ragged
    ("ring_ar", 5, 40009, "fp16", "max"),
    ("rhd_ar", 16, 1 << 18, "int32", "sum"),        # benchmark config 3, scaled down
    ("rhd_ar", 16, 1 << 18, "int32", "min"),
    ("rhd_ar", 6, 100003, "fp32", "sum"),           # part one folds pairs first
    ("mesh_oneshot", 8, 2048, "fp16", "sum"),       # benchmark config 4, 4 KiB
    ("mesh_oneshot", 8, 1 << 21, "fp16", "sum"),    # benchmark config 4, 4 MiB
    ("ring_rs_stage", 7, 1000003, "fp32", "prod"),  # benchmark config 5a, scaled down
    ("ring_rs_stage", 7, 1000003, "int8", "sum"),   # benchmark config 5b, scaled down (odd last slice)
    ("mesh_rs", 7, 999, "int32", "sum"),
    ("nhr_ar", 5, 70001, "bf16", "sum"),
    ("nb_ar", 6, 300007, "int32", "min"),
    ("local_reduce", 8, 100003, "fp32", "sum"),     # stages through the communication buffers
    ("chunk_mesh", 7, 100003, "fp32", "sum"),
    ("ring_ar", 1, 777, "fp32", "sum"),
    ("ring_ar", 3, 0, "fp32", "sum"),
]


def drive(mode, thread, threads, alg, n, count, dtype, op, special=False):
    dt, o = DT[dtype], OPS[op]
    in_count, out_count = buffer_counts(alg, n, count)
    kind = "special" if special else ("prod" if op == "prod" else "default")
    host_in = [gen(dt, in_count, 4000 + 131 * r, kind) for r in range(n)]
    sentinel = gen(dt, out_count, 999, "wide")
    want_in = [x.copy() for x in host_in]
    want_out = [sentinel.copy() for _ in range(n)]
    sb = h.scratch_bytes(ALGS[alg][0], n, count, dt)
    want_scr = [np.full(sb, 0x5A, np.uint8) for _ in range(n)] if sb else None
    with np.errstate(all="ignore"):
        oracle.run(ALGS[alg][1], want_in, want_out, count, dt, o, scratch=want_scr)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_scr = [to_dev(np.full(sb, 0x5A, np.uint8)) for _ in range(n)] if sb else None
    pad = to_dev(np.zeros(256, np.uint8))
    ptr = lambda t: t.data_ptr() if t.numel() else pad.data_ptr()
    bufs = {0: [ptr(t) for t in d_in], 1: [ptr(t) for t in d_out]}
    if sb:
        bufs[2] = [ptr(t) for t in d_scr]
    ops = h.schedule_emit(ALGS[alg][0], n, count, dt)
    replay = caller.Replay(ops, bufs, dt, o)
    prod = op == "prod"   # the primitive refuses PROD like the reference's (cpu_primitives_c_adpt.cc:37) unless told otherwise
    if mode in ("batched", "one_batch"):
        h.HcommGfxThreadSynchronize(thread)
        h.HcommGfxLaunchLogClear(thread)
        code, st = replay.run_batched(thread) if mode == "batched" else replay.run_one_batch(thread)
        if prod and n > 1 and count:
            assert code == h.HcclResult.E_PARA
            return None
        assert code == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        # a step whose operations are of one kind and on 16-byte boundaries is one launch
        if mode == "batched":
            assert st.batches == replay.steps and len(h.launch_log(thread)) >= (replay.steps if count else 0)
        else:
            assert st.batches == 1
    else:
        run = {"threads": replay.run_on_threads, "host_threads": replay.run_on_host_threads,
               "threads_batched": replay.run_on_threads_batched}[mode]
        code, st = run(threads[:n])
        if prod and n > 1 and count:
            assert code == h.HcclResult.E_PARA
            for t in threads[:n]:
                h.HcommGfxThreadSynchronize(t)
            return None
        assert code == 0
        assert h.HcommGfxThreadSynchronize(threads[0]) == 0   # thread 0 joined the others
    strict = op in ("max", "min")
    for r in range(n):
        assert_same(from_dev(d_in[r], host_in[r]), want_in[r], dt, "in[%d]" % r, nan_bits=strict)
        assert_same(from_dev(d_out[r], sentinel), want_out[r], dt, "out[%d]" % r, nan_bits=strict)
        if sb:
            assert np.array_equal(d_scr[r].cpu().numpy(), want_scr[r]), "scratch[%d]" % r
    return st


@pytest.fixture(scope="module")
def rank_threads():
    """Sixteen library-owned threads (streams) with a notify slot per peer."""
    import torch
    assert torch.cuda.is_available()
    code, handles = h.HcommThreadAlloc(h.CommEngine.CPU_TS, 16, 16)
    assert code == 0
    yield handles
    for t in handles:
        h.HcommGfxThreadSynchronize(t)
    h.HcommThreadFree(handles)


@pytest.mark.parametrize("alg,n,count,dtype,op", CASES)
def test_schedule_batched_per_step_matches_oracle(gpu_thread, alg, n, count, dtype, op):
    say("via primitives, batched", alg, n, count, dtype, op)
    drive("batched", gpu_thread, None, alg, n, count, dtype, op)


@pytest.mark.parametrize("alg,n,count,dtype,op", CASES)
def test_schedule_as_one_batch_on_one_thread_matches_oracle(gpu_thread, alg, n, count, dtype, op):
    """Every call of the collective between ONE Start / End pair on one thread: the coalescer keeps apart what touches
    the same memory, so the launches come out step by step."""
    say("via primitives, one batch on one thread", alg, n, count, dtype, op)
    drive("one_batch", gpu_thread, None, alg, n, count, dtype, op)


@pytest.mark.parametrize("alg,n,count,dtype,op", CASES)
def test_schedule_on_one_thread_per_rank_matches_oracle(rank_threads, alg, n, count, dtype, op):
    say("via primitives, one thread per rank", alg, n, count, dtype, op)
    st = drive("threads", None, rank_threads, alg, n, count, dtype, op)
    if st is not None and n > 1 and count:
        assert st.notifies >= 2 * (n - 1)


@pytest.mark.parametrize("alg,n,count,dtype,op", CASES)
def test_schedule_on_one_host_thread_per_rank_matches_oracle(rank_threads, alg, n, count, dtype, op):
    say("via primitives, one host thread per rank", alg, n, count, dtype, op)
    try:
        drive("host_threads", None, rank_threads, alg, n, count, dtype, op)
    finally:
        if (alg, n, count) == CASES[-1][:3]:
            caller.pool_shutdown()


@pytest.mark.parametrize("alg,n,count,dtype,op", CASES)
def test_schedule_as_one_batch_over_a_thread_per_rank_matches_oracle(rank_threads, alg, n, count, dtype, op):
    say("via primitives, one batch over a thread per rank", alg, n, count, dtype, op)
    for t in rank_threads[:n]:
        h.HcommGfxThreadSynchronize(t)
        h.HcommGfxLaunchLogClear(t)
    st = drive("threads_batched", None, rank_threads, alg, n, count, dtype, op)
    if st is None:
        return
    # everything was issued on the first thread of the batch, and in no more launches than one Start / End per step gives
    assert all(not h.launch_log(t) for t in rank_threads[1:n])
    thread = rank_threads[0]
    issued = len(h.launch_log(thread))
    h.HcommGfxLaunchLogClear(thread)
    drive("batched", thread, None, alg, n, count, dtype, op)
    assert issued <= len(h.launch_log(thread))
    if n > 1 and count:   # every record met its wait
        for t in rank_threads[:n]:
            for q in range(n):
                assert h.HcommThreadNotifyWaitOnThread(t, q, 0) == h.HcclResult.E_TIMEOUT


@pytest.mark.parametrize("alg,n,count", [("ring_ar", 8, 70001), ("rhd_ar", 6, 20011), ("mesh_oneshot", 5, 20011)])
@pytest.mark.parametrize("dtype,op", [("fp32", "max"), ("bf16", "min"), ("fp16", "sum")])
def test_special_values_via_primitives(gpu_thread, rank_threads, alg, n, count, dtype, op):
    """Signed zeros, NaNs with per-rank payloads, infinities and denormals through both ways of driving the boundary."""
    say("via primitives, special values", alg, n, count, dtype, op)
    drive("batched", gpu_thread, None, alg, n, count, dtype, op, special=True)
    drive("one_batch", gpu_thread, None, alg, n, count, dtype, op, special=True)
    drive("threads", None, rank_threads, alg, n, count, dtype, op, special=True)
    drive("host_threads", None, rank_threads, alg, n, count, dtype, op, special=True)
    drive("threads_batched", None, rank_threads, alg, n, count, dtype, op, special=True)


def test_repeated_replays_on_threads_leave_no_record_behind(rank_threads):
    """Twenty ring allreduces in a row on eight threads: every record is consumed by its wait, so nothing is left
    pending between collectives and the result is the same every time."""
    for it in range(20):
        drive(("threads", "host_threads", "threads_batched")[it % 3], None, rank_threads, "ring_ar", 8, 65539, "fp32", "sum")
    caller.pool_shutdown()
    for t in rank_threads[:8]:
        for q in range(8):
            assert h.HcommThreadNotifyWaitOnThread(t, q, 0) == h.HcclResult.E_TIMEOUT


@pytest.mark.parametrize("follow", ["eager_call", "synchronize", "callers_stream"])
def test_a_batch_with_notifies_is_ordered_with_eager_work_on_its_threads(rank_threads, follow):
    """The launches of such a batch all go to the stream of its first thread.  What another of its threads was given
    before the batch (eagerly, on its own stream) is finished before the batch reads it, and what it is given after
    the batch starts after the batch's last launch: a chain src -> a (eager, thread 1) -> b (batch, thread 1, posts)
    -> c (batch, thread 0, waits) -> d (after the batch, thread 1) carries src through - whether thread 1 is next
    given a call of the library, is synchronised, or wraps a stream of the caller's that the caller itself queues
    the last copy on."""
    import torch
    say("via primitives, batch with notifies between eager work", follow)
    t0, t1 = rank_threads[:2]
    s1 = None
    if follow == "callers_stream":
        s1 = torch.cuda.Stream()
        code, t1 = h.HcommThreadAllocWithStream(s1.cuda_stream, 4)
        assert code == 0
    nbytes = 1 << 27
    src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda")
    a, b, c, d = (torch.zeros(nbytes, dtype=torch.uint8, device="cuda") for _ in range(4))
    torch.cuda.synchronize()
    try:
        for it in range(3):
            assert h.HcommLocalCopyOnThread(t1, a.data_ptr(), src.data_ptr(), nbytes) == 0
            assert h.HcommBatchModeStart(b"chain") == 0
            assert h.HcommThreadNotifyWaitOnThread(t0, 1, 10) == 0
            assert h.HcommLocalCopyOnThread(t0, c.data_ptr(), b.data_ptr(), nbytes) == 0
            assert h.HcommLocalCopyOnThread(t1, b.data_ptr(), a.data_ptr(), nbytes) == 0
            assert h.HcommThreadNotifyRecordOnThread(t1, t0, 1) == 0
            assert h.HcommBatchModeEnd(b"chain") == 0
            if follow == "eager_call":
                assert h.HcommLocalCopyOnThread(t1, d.data_ptr(), c.data_ptr(), nbytes) == 0
                assert h.HcommGfxThreadSynchronize(t1) == 0
            elif follow == "synchronize":
                assert h.HcommGfxThreadSynchronize(t1) == 0      # thread 1's part of the batch is done when this returns
                d.copy_(c)
                torch.cuda.synchronize()
            else:
                with torch.cuda.stream(s1):
                    d.copy_(c, non_blocking=True)
                s1.synchronize()
            assert torch.equal(d, src), "iteration %d" % it
            assert h.HcommGfxThreadSynchronize(t0) == 0
            src.add_(1)
            for x in (a, b, c, d):
                x.zero_()
            torch.cuda.synchronize()
    finally:
        if s1 is not None:
            h.HcommThreadFreeWithStream([t1])
