"""The symbolic schedule checker: passes every generated schedule (product generator AND oracle trace) and
catches deliberately broken ones - a dropped step, a duplicated contribution, a wrong slice, a race."""
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect

ALL = [(h.Alg.ALLREDUCE_RING, Expect.ALLREDUCE), (h.Alg.REDUCE_SCATTER_RING, Expect.REDUCE_SCATTER_IN_PLACE),
       (h.Alg.ALLREDUCE_RHD, Expect.ALLREDUCE), (h.Alg.ALLREDUCE_MESH_ONESHOT, Expect.ALLREDUCE),
       (h.Alg.REDUCE_SCATTER_MESH, Expect.REDUCE_SCATTER_OUT),
       (h.Alg.REDUCE_SCATTER_RING_STANDALONE, Expect.REDUCE_SCATTER_OUT),
       (h.Alg.ALLREDUCE_MESH_ONESHOT_ASCENDING, Expect.ALLREDUCE),
       (h.Alg.ALLREDUCE_LOCAL_REDUCE, Expect.ALLREDUCE), (h.Alg.ALLREDUCE_CHUNK_MESH, Expect.ALLREDUCE),
       (h.Alg.ALLREDUCE_NHR, Expect.ALLREDUCE), (h.Alg.REDUCE_SCATTER_NHR, Expect.REDUCE_SCATTER_OUT),
       (h.Alg.ALLREDUCE_NB, Expect.ALLREDUCE), (h.Alg.REDUCE_SCATTER_NB, Expect.REDUCE_SCATTER_OUT),
       (h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, Expect.REDUCE_SCATTER_OUT), (h.Alg.ALLREDUCE_DOUBLING, Expect.ALLREDUCE),
       (h.Alg.ALLREDUCE_NHR_ONESHOT, Expect.ALLREDUCE),
       (h.Alg.REDUCE_SCATTER_WINDOW_HALVING, Expect.REDUCE_SCATTER_OUT)]
DENSE_ONLY = (h.Alg.REDUCE_SCATTER_LOCAL_REDUCE,)


@pytest.mark.parametrize("alg,expect", ALL)
def test_generated_schedules_pass(alg, expect):
    for n in list(range(1, 18)) + [24, 31, 32]:
        if alg == h.Alg.ALLREDUCE_DOUBLING and n & (n - 1):
            continue
        if alg == h.Alg.ALLREDUCE_LOCAL_REDUCE and n & (n - 1) and n != 3:   # the counts whose folds land
            continue
        for count, dt, unit in ((0, h.HcommDataType.FP32, 4), (1, h.HcommDataType.INT8, 1),
                                (1000, h.HcommDataType.FP16, 2), (100003, h.HcommDataType.FP32, 4),
                                (1200007, h.HcommDataType.FP32, 4)):
            assert h.schedule_check(alg, n, count, dt)[:2] == (0, 0), (alg, n, count)
            ops = oracle.trace(alg, n, count, dt)        # the oracle's per-rank programs pass the same check
            assert h.oplist_check(ops, n, expect, count, unit)[:2] == (0, 0), (alg, n, count)
            if expect == Expect.REDUCE_SCATTER_OUT and alg not in DENSE_ONLY:
                assert h.schedule_check(alg, n, count, dt, stride=count + 77)[:2] == (0, 0)


def test_benchmark_configurations_pass_at_full_size():
    assert h.schedule_check(h.Alg.ALLREDUCE_RING, 8, 67108864, h.HcommDataType.BFP16)[:2] == (0, 0)
    assert h.schedule_check(h.Alg.ALLREDUCE_RHD, 16, 33554432, h.HcommDataType.INT32)[:2] == (0, 0)
    assert h.schedule_check(h.Alg.REDUCE_SCATTER_RING, 7, 100000003, h.HcommDataType.INT8)[:2] == (0, 0)
    assert h.schedule_check(h.Alg.ALLREDUCE_MESH_ONESHOT, 8, 2097152, h.HcommDataType.FP16)[:2] == (0, 0)


def ring(n=4, count=1024):
    return h.schedule_emit(h.Alg.ALLREDUCE_RING, n, count, h.HcommDataType.FP32), n, count


def test_dropped_operation_is_a_semantic_error():
    ops, n, count = ring()
    for victim in (0, 5, len(ops) - 1):
        broken = ops[:victim] + ops[victim + 1:]
        c, s, msg = h.oplist_check(broken, n, Expect.ALLREDUCE, count, 4)
        assert c == 0 and s > 0 and "rank" in msg


def test_duplicated_contribution_is_a_semantic_error():
    ops, n, count = ring()
    first_reduce = [o for o in ops if o[1] == 1][0]
    # the same reduce once more, in a step of its own right after step 0
    broken = [((o[0] + 1 if o[0] >= 1 else 0),) + o[1:] for o in ops] + [(1,) + first_reduce[1:]]
    broken.sort(key=lambda o: (o[0], o[2]))
    c, s, msg = h.oplist_check(broken, n, Expect.ALLREDUCE, count, 4)
    assert s > 0 and "wrong number of times" in msg


def test_wrong_slice_offset_is_a_semantic_error():
    ops, n, count = ring()
    k = [i for i, o in enumerate(ops) if o[1] == 1][3]
    step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes = ops[k]
    other = [o for o in ops if o[1] == 1 and o[7] != soff][0][7]
    broken = list(ops)
    broken[k] = (step, kind, rank, dbuf, doff, srank, sbuf, other, nbytes)     # reads a different slice of the peer
    c, s, msg = h.oplist_check(broken, n, Expect.ALLREDUCE, count, 4)
    assert s > 0


def test_race_inside_a_step_is_a_conflict():
    ops, n, count = ring()
    # merge step 1 into step 0: rank r now reads what rank r-1 writes in the same step
    merged = [((0 if o[0] == 1 else o[0]),) + o[1:] for o in ops]
    merged.sort(key=lambda o: (o[0], o[2]))
    c, s, msg = h.oplist_check(merged, n, Expect.ALLREDUCE, count, 4)
    assert c > 0 and "step 0" in msg
    # two writers of one range
    ops2 = list(ops)
    step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes = ops2[0]
    ops2.insert(1, (step, kind, rank, dbuf, doff, (srank + 1) % n, sbuf, soff, nbytes))
    c, s, msg = h.oplist_check(ops2, n, Expect.ALLREDUCE, count, 4)
    assert c > 0


def test_reduce_scatter_expectations_are_distinguished():
    n, count = 4, 256
    ops = h.schedule_emit(h.Alg.REDUCE_SCATTER_MESH, n, count, h.HcommDataType.FP32)
    assert h.oplist_check(ops, n, Expect.REDUCE_SCATTER_OUT, count, 4)[:2] == (0, 0)
    assert h.oplist_check(ops, n, Expect.ALLREDUCE, count, 4)[1] > 0          # it is not an allreduce
    swapped = [o[:7] + (((o[7] // (count * 4) + 1) % n) * count * 4, o[8]) if o[1] == 0 else o for o in ops]
    assert h.oplist_check(swapped, n, Expect.REDUCE_SCATTER_OUT, count, 4)[1] > 0   # output took the wrong slice


def test_argument_checks():
    import ctypes as C
    from hcomm_amd import api as raw
    rep = h.CheckReport()
    assert raw._oplist_check(None, 0, 4, 0, 10, 0, 4, None) == h.HcclResult.E_PTR
    assert raw._oplist_check(None, 3, 4, 0, 10, 0, 4, C.byref(rep)) == h.HcclResult.E_PTR
    assert raw._oplist_check(None, 0, 0, 0, 10, 0, 4, C.byref(rep)) == h.HcclResult.E_PARA
    assert raw._oplist_check(None, 0, 4, 9, 10, 0, 4, C.byref(rep)) == h.HcclResult.E_PARA
    bad = [(0, 1, 7, 0, 0, 0, 0, 0, 16)]                                       # rank out of range
    with pytest.raises(h.HcommError):
        h.oplist_check(bad, 4, Expect.ALLREDUCE, 10, 4)
