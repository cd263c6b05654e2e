"""The reduction trees of the single-launch lowerings, read back from the plans, against the expression trees a
symbolic replay of the ORACLE's operation list leaves in the outputs (a different generator from the product's), and
against the hand-derived trees of the golden file.  No GPU: plans are built on made-up addresses."""
import json
import os

import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import HcclResult as R

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "schedules_hand_derived.json")))
BASE = 0x7f0000000000


def ptrs(n):
    ins = [BASE + r * (1 << 32) for r in range(n)]
    outs = [BASE + (64 + r) * (1 << 32) for r in range(n)]
    return ins, outs, {p: r for r, p in enumerate(ins)}


def output_trees(ops, n):
    """{(offset, bytes): tree} of rank 0's output after a symbolic replay; asserts that every rank's output holds the
    same trees.  A leaf is (rank, input offset); a fold is [dst, src]."""
    cells = {}
    for step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes in ops:
        if nbytes == 0:
            continue
        skey, dkey = (srank, sbuf, soff, nbytes), (rank, dbuf, doff, nbytes)
        if skey not in cells:
            assert sbuf == 0, "read of a range that was never written with these bounds"
            cells[skey] = (srank, soff)
        assert dbuf != 0 or not kind or dkey in cells or True
        if kind:
            if dkey not in cells:
                assert dbuf == 0
                cells[dkey] = (rank, doff)
            cells[dkey] = [cells[dkey], cells[skey]]
        else:
            cells[dkey] = cells[skey]
    per_rank = [{(k[2], k[3]): v for k, v in cells.items() if k[0] == r and k[1] == 1} for r in range(n)]
    return per_rank


def strip(tree, off):
    """(rank, offset) leaves -> rank, checking that every leaf is read at the segment's own offset."""
    if isinstance(tree, tuple):
        assert tree[1] == off
        return tree[0]
    return [strip(tree[0], off), strip(tree[1], off)]


def plan_segments(plan, rank_of):
    out = {}
    for i, rec in enumerate(plan.launches()):
        assert rec.kind == h.Kernel.TREE
        for s in range(rec.nseg):
            tree, off, nbytes = h.plan_tree(plan, i, s, rank_of)
            out[(off, nbytes)] = tree
    return out


@pytest.mark.parametrize("n", [2, 3, 4, 8, 16, 32])
@pytest.mark.parametrize("count,dtype", [(1 << 20, oracle.F32), (300007 * 16, oracle.BF16), (32 * 16384 + 40, oracle.I8)])
def test_deterministic_mesh_allreduce_single_launch_trees_equal_the_replay(n, count, dtype):
    ins, outs, rank_of = ptrs(n)
    plan = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, ins, outs, count, dtype, oracle.SUM)
    try:
        got = plan_segments(plan, rank_of)
        per_rank = output_trees(oracle.trace(oracle.ALG_ALLREDUCE_LOCAL_REDUCE, n, count, dtype), n)
        for r in range(1, n):
            assert per_rank[r] == per_rank[0]
        want = {k: strip(v, k[0]) for k, v in per_rank[0].items()}
        assert got == want
        unit = h.DTYPE_SIZE[dtype]
        assert sum(b for _, b in got) == count * unit
        assert plan.info.movedBytes == 2 * n * count * unit      # n reads and n writes per element, nothing else
    finally:
        plan.destroy()


def test_deterministic_mesh_allreduce_single_launch_trees_hand_derived():
    for n_s, trees in GOLD["local_reduce_slice_tree"].items():
        n = int(n_s)
        ins, outs, rank_of = ptrs(n)
        count = n * 4096 * 4 + 5000                              # 16 KiB slots, ragged last slice
        plan = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, ins, outs, count, oracle.F32, oracle.SUM)
        got = plan_segments(plan, rank_of)
        per = h.scratch_bytes(h.Alg.ALLREDUCE_LOCAL_REDUCE, n, count, oracle.F32) // n
        assert {off // per: t for (off, _), t in got.items()} == {int(d): t for d, t in trees.items()}
        plan.destroy()


def test_deterministic_mesh_allreduce_single_launch_limits():
    ins, outs, _ = ptrs(32)
    # 32 ranks: trees of depth 6 over 64 leaf positions, four segments' tables per launch, so 8 launches for 32 slices
    p = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, ins, outs, 1 << 22, oracle.F32, oracle.SUM)
    assert [(r.kind, r.nseg) for r in p.launches()] == [(h.Kernel.TREE, 4)] * 8
    p.destroy()
    ins, outs, _ = ptrs(4)
    with pytest.raises(h.HcommError) as e:                       # slots of 10 bytes: slices off 16-byte boundaries
        h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, ins, outs, 38, oracle.I8, oracle.SUM)
    assert e.value.code == R.E_NOT_SUPPORT
    with pytest.raises(h.HcommError) as e:                       # as the step-wise replay: rank counts whose folds land
        h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, ptrs(5)[0], ptrs(5)[1], 4096, oracle.F32, oracle.SUM)
    assert e.value.code == R.E_PARA
    p = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, ins[:1], outs[:1], 4096, oracle.F32, oracle.SUM)
    assert [r.kind for r in p.launches()] == [h.Kernel.COPY]
    p.destroy()
    p = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.FUSED, ins, outs, 0, oracle.F32, oracle.SUM)
    assert p.launches() == []
    p.destroy()


@pytest.mark.parametrize("n", [2, 3, 4, 5, 6, 7, 8, 12, 16, 17, 31, 32])
def test_deterministic_mesh_reduce_scatter_single_launch_trees_equal_the_replay(n):
    ins, outs, rank_of = ptrs(n)
    count, dtype = 4096, oracle.F32
    plan = h.Plan(h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, h.Lowering.FUSED, ins, outs, count, dtype, oracle.SUM)
    try:
        got = plan_segments(plan, rank_of)
        per_rank = output_trees(oracle.trace(oracle.ALG_RS_LOCAL_REDUCE, n, count, dtype), n)
        for d in range(n):
            assert list(per_rank[d]) == [(0, count * 4)]
            assert got[(d * count * 4, count * 4)] == strip(per_rank[d][(0, count * 4)], d * count * 4), d
        if str(n) in GOLD["rs_local_reduce_rank_tree"]:
            for d_s, tree in GOLD["rs_local_reduce_rank_tree"][str(n)].items():
                assert got[(int(d_s) * count * 4, count * 4)] == tree
    finally:
        plan.destroy()


@pytest.mark.parametrize("alg,oalg", [(h.Alg.ALLREDUCE_NHR, oracle.ALG_ALLREDUCE_NHR), (h.Alg.ALLREDUCE_NB, oracle.ALG_ALLREDUCE_NB),
                                      (h.Alg.ALLREDUCE_NHR_ONESHOT, oracle.ALG_ALLREDUCE_NHR_ONESHOT)])
@pytest.mark.parametrize("n", [2, 3, 5, 6, 8, 13, 16, 32])
def test_rotation_tree_launches_equal_the_replay(alg, oalg, n):
    """The same read-back for the older tree lowerings (their launches also store partials into the inputs, which
    the replayed outputs do not show; the GPU tests compare those)."""
    ins, outs, rank_of = ptrs(n)
    count, dtype = 100003, oracle.F32
    plan = h.Plan(alg, h.Lowering.FUSED, ins, outs, count, dtype, oracle.SUM)
    try:
        got = plan_segments(plan, rank_of)
        per_rank = output_trees_in_place(oracle.trace(oalg, n, count, dtype), n)
        for r in range(n):
            assert merged_runs(per_rank[r]) == merged_runs(got), r
    finally:
        plan.destroy()


@pytest.mark.parametrize("n", [2, 4, 8, 16, 32])
def test_halving_tree_launch_equals_the_replay(n):
    """Recursive halving-doubling on a power-of-two rank count (with other counts the launch first absorbs the odd
    neighbours, which this read-back does not show; the GPU tests cover them)."""
    ins, outs, rank_of = ptrs(n)
    plan = h.Plan(h.Alg.ALLREDUCE_RHD, h.Lowering.FUSED, ins, outs, 100003, oracle.F32, oracle.SUM)
    try:
        per_rank = output_trees_in_place(oracle.trace(oracle.ALG_ALLREDUCE_RHD, n, 100003, oracle.F32), n)
        for r in range(n):
            assert merged_runs(per_rank[r]) == merged_runs(plan_segments(plan, rank_of)), r
    finally:
        plan.destroy()


@pytest.mark.parametrize("n", [2, 4, 8, 16, 32])
def test_recursive_doubling_keep_inputs_launch_holds_every_ranks_own_tree(n):
    """Whole-message recursive doubling: rank r's output is the tree whose position q holds rank r XOR q; the schedule
    writes the inputs on the way, the single launch (inputs kept) reads only the originals."""
    ins, outs, rank_of = ptrs(n)
    count = 25000
    plan = h.Plan(h.Alg.ALLREDUCE_DOUBLING, h.Lowering.FUSED_KEEP_INPUTS, ins, outs, count, oracle.F32, oracle.SUM)
    try:
        per_rank = output_trees_in_place(oracle.trace(oracle.ALG_ALLREDUCE_DOUBLING, n, count, oracle.F32), n)
        seen = set()
        for i, rec in enumerate(plan.launches()):
            assert rec.kind == h.Kernel.TREE
            for sg in range(rec.nseg):
                tree, off, nbytes, owner = h.plan_tree(plan, i, sg, rank_of, with_owner=True)
                assert (off, nbytes) == (0, count * 4) and owner not in seen
                seen.add(owner)
                assert per_rank[owner] == {(0, count * 4): tree}, owner
                x = [owner ^ q for q in range(n)]
                step = 1
                while step < n:
                    for q in range(0, n, 2 * step):
                        x[q] = [x[q], x[q + step]]
                    step *= 2
                assert tree == x[0]
        assert seen == set(range(n))
        assert plan.info.movedBytes == (n + 1) * n * count * 4
    finally:
        plan.destroy()
    with pytest.raises(h.HcommError) as e:          # the lowering that reproduces the inputs' final contents has none
        h.Plan(h.Alg.ALLREDUCE_DOUBLING, h.Lowering.FUSED, ins, outs, count, oracle.F32, oracle.SUM)
    assert e.value.code == R.E_NOT_SUPPORT


OPLIST_CASES = [
    # oracle algorithm, ranks: schedules whose trees are at most 5 folds deep and whose ranges keep their bounds
    (oracle.ALG_ALLREDUCE_RING, 2), (oracle.ALG_ALLREDUCE_RING, 4), (oracle.ALG_ALLREDUCE_RING, 6),
    (oracle.ALG_ALLREDUCE_MESH_ONESHOT, 3), (oracle.ALG_ALLREDUCE_MESH_ONESHOT, 6), (oracle.ALG_ALLREDUCE_MESH_ASCENDING, 5),
    (oracle.ALG_ALLREDUCE_LOCAL_REDUCE, 8), (oracle.ALG_ALLREDUCE_LOCAL_REDUCE, 16),
    (oracle.ALG_ALLREDUCE_DOUBLING, 8), (oracle.ALG_ALLREDUCE_NHR_ONESHOT, 7), (oracle.ALG_ALLREDUCE_NB, 6),
]


@pytest.mark.parametrize("oalg,n", OPLIST_CASES)
def test_any_op_list_with_shallow_trees_lowers_to_tree_launches(oalg, n):
    """HcommGfxPlanCreateFromOpsKeepInputs on the oracle's operation lists: the launches' trees are the replay's."""
    ins, outs, rank_of = ptrs(n)
    count = 6 * 8192 * 5
    ops = oracle.trace(oalg, n, count, oracle.F32)
    plan = h.OpListKeepInputsPlan(ops, ins, outs, oracle.F32, oracle.SUM)
    try:
        if oalg == oracle.ALG_ALLREDUCE_LOCAL_REDUCE:     # slots at other offsets than the slices: the exact-cell replay
            per_rank = [{k: strip(v, k[0]) for k, v in cells.items()} for cells in output_trees(ops, n)]
        else:
            per_rank = output_trees_in_place(ops, n)
        got = [{} for _ in range(n)]
        for i, rec in enumerate(plan.launches()):
            assert rec.kind == h.Kernel.TREE
            for sg in range(rec.nseg):
                tree, off, nbytes, owner = h.plan_tree(plan, i, sg, rank_of, with_owner=True)
                for r in (range(n) if owner < 0 else [owner]):
                    assert (off, nbytes) not in got[r]
                    got[r][(off, nbytes)] = tree
        for r in range(n):
            assert merged_runs(got[r]) == merged_runs(per_rank[r]), r
    finally:
        plan.destroy()


def test_op_lists_the_tree_lowering_refuses():
    ins, outs, _ = ptrs(8)
    for oalg, n in ((oracle.ALG_ALLREDUCE_RING, 8),          # chains of 7 folds
                    (oracle.ALG_ALLREDUCE_RHD, 8),           # halving steps fold several slices as one range
                    (oracle.ALG_ALLREDUCE_CHUNK_MESH, 4),    # copies the whole message, then folds sub-chunks of it
                    (oracle.ALG_RS_MESH, 4)):                # slice r of every input lands at offset 0 of out[r]
        with pytest.raises(h.HcommError) as e:
            h.OpListKeepInputsPlan(oracle.trace(oalg, n, 1 << 18, oracle.F32), ins[:n], outs[:n], oracle.F32, oracle.SUM)
        assert e.value.code == R.E_NOT_SUPPORT, oalg
    with pytest.raises(h.HcommError) as e:                   # a value read that the list never wrote
        h.OpListKeepInputsPlan([(0, 0, 0, 1, 0, 1, 2, 0, 4096)], ins[:2], outs[:2], oracle.F32, oracle.SUM)
    assert e.value.code == R.E_NOT_SUPPORT
    with pytest.raises(h.HcommError) as e:                   # a user-buffer role of the op-base lists
        h.OpListKeepInputsPlan([(0, 0, 0, 1, 0, 1, 3, 0, 4096)], ins[:2], outs[:2], oracle.F32, oracle.SUM)
    assert e.value.code == R.E_PARA
    # Operations of one step that observe each other have no single meaning (the step-wise lowering runs them one
    # after the other, the symbolic replay gives all of them the state the step began with): refused, not guessed.
    swap = [(0, 0, 0, 1, 0, 0, 0, 0, 4096), (0, 0, 1, 1, 0, 1, 0, 0, 4096),
            (1, 1, 0, 1, 0, 1, 1, 0, 4096), (1, 1, 1, 1, 0, 0, 1, 0, 4096)]          # out0 += out1 beside out1 += out0
    twice = [(0, 0, 0, 1, 0, 0, 0, 0, 4096),
             (1, 1, 0, 1, 0, 1, 0, 0, 4096), (1, 1, 0, 1, 0, 2, 0, 0, 4096)]         # out0 += in1 beside out0 += in2
    for ops, n in ((swap, 2), (twice, 3)):
        with pytest.raises(h.HcommError) as e:
            h.OpListKeepInputsPlan(ops, ins[:n], outs[:n], oracle.F32, oracle.SUM)
        assert e.value.code == R.E_NOT_SUPPORT
    # the same two folds in steps of their own are a chain of two: out0 = (in0 + in1) + in2
    p = h.OpListKeepInputsPlan([twice[0], twice[1], (2,) + twice[2][1:]], ins[:3], outs[:3], oracle.F32, oracle.SUM)
    rank_of = {ins[r]: r for r in range(3)}
    assert h.plan_tree(p, 0, 0, rank_of)[0] == [[0, 1], 2]
    p.destroy()


def test_deep_or_self_referencing_lists_are_refused_at_once():
    """Trees deeper than the kernel folds are refused while the list is replayed, not after: a value folded into itself
    doubles its tree with every operation and a chain grows by one fold per operation, so both lists below would
    otherwise cost time or stack in proportion to 2^n / n."""
    import time
    ins, outs, _ = ptrs(2)
    first = (0, 0, 0, 1, 0, 0, 0, 0, 4096)                                           # out0 = in0
    doubling = [first] + [(1 + i, 1, 0, 1, 0, 0, 1, 0, 4096) for i in range(64)]       # out0 += out0, 64 times
    chain = [first] + [(1 + i, 1, 0, 1, 0, 1, 0, 0, 4096) for i in range(200000)]      # out0 += in1, 200,000 times
    for ops in (doubling, chain):
        t0 = time.perf_counter()
        with pytest.raises(h.HcommError) as e:
            h.OpListKeepInputsPlan(ops, ins, outs, oracle.F32, oracle.SUM)
        assert e.value.code == R.E_NOT_SUPPORT
        assert time.perf_counter() - t0 < 5.0


def merged_runs(segments):
    """[(lo, hi, tree)] with neighbours that hold the same tree joined: independent of how the bytes were cut."""
    out = []
    for (off, nbytes), tree in sorted(segments.items()):
        if out and out[-1][1] == off and out[-1][2] == tree:
            out[-1] = (out[-1][0], off + nbytes, tree)
        else:
            out.append((off, off + nbytes, tree))
    return out


def output_trees_in_place(ops, n):
    """As output_trees for schedules that reduce inside the input buffers and whose steps run in parallel: reads see
    the state before the step; ranges are tracked per byte span so that a gather of several slices at once resolves."""
    state = {}                                                   # (rank, buf) -> sorted list of [lo, hi, tree, lo0]
    def read(rank, buf, off, nbytes):
        out, pos = [], off
        for lo, hi, tree in sorted(state.get((rank, buf), [])):
            if hi <= off or lo >= off + nbytes:
                continue
            assert lo >= pos or lo <= off
            if lo > pos:
                assert buf == 0
                out.append((pos, lo, ("in", rank)))
            out.append((max(lo, off), min(hi, off + nbytes), tree))
            pos = min(hi, off + nbytes)
        if pos < off + nbytes:
            assert buf == 0, "read of unwritten memory"
            out.append((pos, off + nbytes, ("in", rank)))
        return out
    def write(rank, buf, pieces):
        cur = state.setdefault((rank, buf), [])
        for lo, hi, tree in pieces:
            nxt = []
            for a, b, t in cur:
                if b <= lo or a >= hi:
                    nxt.append((a, b, t))
                else:
                    if a < lo:
                        nxt.append((a, lo, t))
                    if b > hi:
                        nxt.append((hi, b, t))
            nxt.append((lo, hi, tree))
            cur[:] = nxt
    by_step = {}
    for o in ops:
        by_step.setdefault(o[0], []).append(o)
    for step in sorted(by_step):
        pending = []
        for _, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes in by_step[step]:
            if nbytes == 0:
                continue
            src = read(srank, sbuf, soff, nbytes)
            if kind:
                dst = read(rank, dbuf, doff, nbytes)
                cuts = sorted({p for lo, hi, _ in src for p in (lo - soff, hi - soff)} | {p for lo, hi, _ in dst for p in (lo - doff, hi - doff)})
                pieces = []
                for a, b in zip(cuts, cuts[1:]):
                    s = [t for lo, hi, t in src if lo - soff <= a and b <= hi - soff][0]
                    d = [t for lo, hi, t in dst if lo - doff <= a and b <= hi - doff][0]
                    pieces.append((doff + a, doff + b, ("f", d, s, doff - soff)))
                pending.append((rank, dbuf, pieces))
            else:
                pending.append((rank, dbuf, [(lo - soff + doff, hi - soff + doff, ("m", t, doff - soff)) for lo, hi, t in src]))
        for rank, dbuf, pieces in pending:
            write(rank, dbuf, pieces)
    def simplify(t):
        if t[0] == "in":
            return t[1]
        if t[0] == "m":
            assert t[2] == 0, "a copy between different offsets"
            return simplify(t[1])
        assert t[3] == 0
        return [simplify(t[1]), simplify(t[2])]
    per_rank = []
    for r in range(n):
        merged = {}
        for lo, hi, t in sorted(state.get((r, 1), [])):
            merged[(lo, hi - lo)] = simplify(t)
        per_rank.append(merged)
    return per_rank


# ---- the AICPU deterministic reduce-scatter: SelfLocalReduce's folds as the rank-order tree -----------------------

def window_halving_tree(n):
    """TaskOrchestrator::SelfLocalReduce (aicpu_kfc/algorithm/task_orchestrator.cc:719-755) on symbols: slot s holds
    rank s's slice; the slots beyond the largest power of two fold onto the first ones, then halving rounds."""
    slots = list(range(n))
    p = 1 << (n.bit_length() - 1)
    for i in range(n - p):
        slots[i] = [slots[i], slots[p + i]]
    h_ = p // 2
    while h_ >= 1:
        for i in range(h_):
            slots[i] = [slots[i], slots[h_ + i]]
        h_ //= 2
    return slots[0]


@pytest.mark.parametrize("n", [2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17, 24, 31, 32])
def test_window_halving_single_launch_is_the_rank_order_tree(n):
    gold = GOLD["window_halving_rank_tree"]
    if str(n) in gold:
        assert window_halving_tree(n) == gold[str(n)]
    ins, outs, rank_of = ptrs(n)
    for count, stride in ((4096, 0), (1000, 1000 + 24)):
        plan = h.Plan(h.Alg.REDUCE_SCATTER_WINDOW_HALVING, h.Lowering.FUSED, ins, outs, count, oracle.F32, oracle.SUM, stride)
        try:
            recs = plan.launches()
            assert [r.kind for r in recs] == [h.Kernel.TREE] and recs[0].nseg == n
            pitch = (stride or count) * 4
            for d in range(n):
                tree, off, nbytes, owner = h.plan_tree(plan, 0, d, rank_of, with_owner=True)
                assert (tree, off, nbytes, owner) == (window_halving_tree(n), d * pitch, count * 4, d)
            assert plan.info.movedBytes == (n + 1) * n * count * 4       # n reads and one write per output element
            assert plan.info.algorithmicBytes == oracle.algorithmic_bytes(oracle.ALG_RS_WINDOW_HALVING, n, count, oracle.F32)
        finally:
            plan.destroy()
    with pytest.raises(h.HcommError) as e:                               # blocks off 16-byte boundaries: step-wise only
        h.Plan(h.Alg.REDUCE_SCATTER_WINDOW_HALVING, h.Lowering.FUSED, ins, outs, 1001, oracle.F32, oracle.SUM, 1003)
    assert e.value.code == R.E_NOT_SUPPORT
