"""AllReduceLocalReduce for rank counts that are not powers of two, settled without a GPU.

The reference's template (src/legacy/ascend910/algorithm/base/alg_template/temp_all_reduce/all_reduce_local_reduce.cc)
has a loop for the slots beyond the power-of-two block (:311-327), so it means to take any rank count.  Replaying its
statements - where every round's data lands (:222-266), which slots every fold combines (:301-364), which slot the
gather fetches (:419) - shows that the folded slice ends up where the gather reads it for n = 2^k and n = 3 only; for
every other count some rank's gather source is a slot that holds a partial sum.  Three witnesses that do not share
code: a restatement of the slot arithmetic in Python below, the library's symbolic schedule checker run over the
oracle's statement-by-statement trace, and the closed form of the library's own generator."""
import numpy as np
import pytest

import hcomm_amd as h
import oracle
from hcomm_amd import HcclResult as R


def replay_slots(n):
    """For every rank d: ({slot: set of contributing ranks} after RunReduceScatter + RunLocalReduce, slot the gather
    reads).  Slots are indices inside d's window; a window has n - 1 slots."""
    out = []
    for d in range(n):
        slot = {}
        own = d - 1 if d == n - 1 else d                       # :233, and :197-199 (natural offset = slot d, window one up for the last rank :102-110)
        slot[own] = {d}
        for rnd in range(1, n):                                # the round in which rank d is some sender's dstRank (:222-226)
            sender = (d - rnd) % n
            w = (d + rnd) % (n - 1)
            if d == n - 1:
                w = (w + n - 2) % (n - 1)
            if rnd == n - 1:
                slot[own] = slot[own] | {sender}               # :229-250 reduce into the own slot
            else:
                assert w not in slot
                slot[w] = {sender}                             # :251-266 copy
        assert sorted(slot) == list(range(n - 1))
        power = int(np.floor(np.log2(n - 1))) if n > 2 else 0
        block = 1 << power
        for i in range(n - block - 1):                         # :311-327
            if d < block:
                slot[i] = slot[i] | slot[block + i]
            else:
                slot[block + i] = slot[block + i] | slot[i]
        center = d if d < block else d - block + 1             # :328-331
        center = min(center, block - 1)
        first = 0 if d < block else n - block - 1
        for rnd in range(power):                               # :333-362
            h_ = block >> (rnd + 1)
            if center < h_:
                for i in range(h_):
                    slot[first + i] = slot[first + i] | slot[first + h_ + i]
            else:
                for i in range(h_):
                    slot[first + h_ + i] = slot[first + h_ + i] | slot[first + i]
                first += h_
                center -= h_
        out.append((slot, n - 2 if d == n - 1 else d))         # :419: offset dstRank * slices_[0].size of the peer's buffer
    return out


LANDS = {2, 3, 4, 8, 16, 32}


@pytest.mark.parametrize("n", range(2, 33))
def test_where_the_folded_slice_lands(n):
    complete = all(slot[read] == set(range(n)) for slot, read in replay_slots(n))
    assert complete == (n in LANDS)
    if n in (5, 6, 7):      # the complete sum exists in every window, but for these ranks not in the slot the gather fetches
        missed = [d for d, (slot, read) in enumerate(replay_slots(n)) if slot[read] != set(range(n))]
        assert missed == {5: [4], 6: [4, 5], 7: [4, 5]}[n]
        assert all(any(v == set(range(n)) for v in slot.values()) for slot, _ in replay_slots(n))


@pytest.mark.parametrize("n", [2, 3, 4, 5, 6, 7, 8, 9, 12, 16])
def test_checker_on_the_statements_as_written(n):
    """The oracle's per-rank program follows the template statement by statement for any n; the library's symbolic
    checker (every output range = every rank exactly once) accepts the trace exactly where the replay above lands."""
    ops = oracle.trace(oracle.ALG_ALLREDUCE_LOCAL_REDUCE_AS_WRITTEN, n, 30000, oracle.F32)
    conflicts, wrong, _ = h.oplist_check(ops, n, h.Expect.ALLREDUCE, 30000, 4)
    assert conflicts == 0
    assert (wrong == 0) == (n in LANDS)


@pytest.mark.parametrize("n", range(1, 33))
def test_library_takes_exactly_the_counts_that_land(n):
    try:
        ops = h.schedule_emit(h.Alg.ALLREDUCE_LOCAL_REDUCE, n, 30000, oracle.F32)
        code = R.SUCCESS
    except h.HcommError as e:
        ops, code = None, e.code
    if n == 1 or n in LANDS:
        assert code == R.SUCCESS
        assert h.oplist_check(ops, n, h.Expect.ALLREDUCE, 30000, 4)[:2] == (0, 0)
        assert sorted(ops) == sorted(oracle.trace(oracle.ALG_ALLREDUCE_LOCAL_REDUCE, n, 30000, oracle.F32))
    else:
        assert code == R.E_PARA


def test_three_ranks_fold_trees_in_the_single_launch():
    """n = 3 through the tree lowering: slice d = (in[d] (op) in[d+1]) (op) in[d+2], as derived by hand."""
    n, count = 3, 3 * 4096 * 4 + 5000
    ins = [0x10000000 * (r + 1) for r in range(n)]
    outs = [(1 << 36) + 0x10000000 * (r + 1) for r in range(n)]
    plan = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, ins, outs, count, oracle.F32, oracle.SUM)
    rank_of = {ins[r]: r for r in range(n)}
    trees = {}
    for i, rec in enumerate(plan.launches()):
        for sg in range(rec.nseg):
            tree, off, nbytes = h.plan_tree(plan, i, sg, rank_of)[:3]
            trees[off] = tree
    per = h.scratch_bytes(h.Alg.ALLREDUCE_LOCAL_REDUCE, n, count, oracle.F32) // n
    assert trees == {0: [[0, 1], 2], per: [[1, 2], 0], 2 * per: [[2, 0], 1]}
    plan.destroy()
