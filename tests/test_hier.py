"""The ring executor's three-step allreduce over two communicator levels (reduce-scatter inside a server, allreduce
between the servers on the own segment, all-gather inside the server): the oracle's per-rank transcription against
hand-derived operation lists and reduction trees, against exact integer arithmetic, against the symbolic checker and
against the product's generator, which composes the three levels from its flat schedules instead."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))["hier_allreduce"]
LEVEL1 = [oracle.ALG_ALLREDUCE_RING, oracle.ALG_ALLREDUCE_RHD, oracle.ALG_ALLREDUCE_NHR, oracle.ALG_ALLREDUCE_NB]
SHAPES = [(2, 8), (4, 8), (3, 5), (1, 8), (8, 1), (2, 2), (4, 4), (5, 3), (2, 16), (1, 1)]


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["ops_2x2_ring_fp32_count100"]["ops"]]
    assert oracle.trace_hier(oracle.ALG_ALLREDUCE_RING, 2, 2, 100, oracle.F32) == want
    assert h.hier_emit(h.Alg.ALLREDUCE_RING, 2, 2, 100, oracle.F32) == want


def test_mesh_level0_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["mesh_rank0_ops_1x4_fp32_count384"]["ops"]]
    for gen in (oracle.trace_hier, h.hier_emit):
        got = [o for o in gen(oracle.ALG_ALLREDUCE_RING, 1, 4, 384, oracle.F32, mesh=True) if o[2] == 0]
        assert got == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_mesh_level0_reduction_trees_hand_derived(op):
    ins = order_sensitive_inputs(4, 384, op, seed=310)
    work = [x.copy() for x in ins]
    outs = [np.zeros(384, np.float32) for _ in range(4)]
    oracle.run_hier(oracle.ALG_ALLREDUCE_RING, 1, 4, work, outs, 384, oracle.F32, op, mesh=True)
    for first, cnt, tree in GOLD["mesh_trees_1x4_fp32_count384"]["pieces"]:
        want = eval_tree(tree, [x[first:first + cnt] for x in ins], op)
        for r in range(4):
            assert np.array_equal(outs[r][first:first + cnt].view(np.uint32), want.view(np.uint32)), (first, r)


def test_mesh_stream_pieces_hand_derived():
    """A ragged last segment of 1000 bytes cut for 3 and for 7 streams (the fixture places it at offset 2048)."""
    c = GOLD["mesh_stream_pieces"]
    for n, key in ((4, "streams3"), (8, "streams7")):
        count = next(k for k in range(1, 40000) if oracle.slices_ring(k, 1, n)[n - 1][1] == c["seg"][1])
        seg = oracle.slices_ring(count, 1, n)[n - 1]
        for gen in (oracle.trace_hier, h.hier_emit):
            ops = [o for o in gen(oracle.ALG_ALLREDUCE_RING, 1, n, count, oracle.I8, mesh=True) if o[0] == 0 and o[2] == n - 1]
            assert [[o[4] - seg[0] + c["seg"][0], o[8]] for o in ops] == c[key], (n, count)


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_reduction_trees_hand_derived(op):
    ins = order_sensitive_inputs(6, 192, op, seed=300)
    work = [x.copy() for x in ins]
    outs = [np.zeros(192, np.float32) for _ in range(6)]
    oracle.run_hier(oracle.ALG_ALLREDUCE_RING, 2, 3, work, outs, 192, oracle.F32, op)
    for first, cnt, tree in GOLD["trees_2x3_ring_fp32_count192"]["pieces"]:
        want = eval_tree(tree, [x[first:first + cnt] for x in ins], op)
        for r in range(6):
            assert np.array_equal(outs[r][first:first + cnt].view(np.uint32), want.view(np.uint32)), (first, r)


def test_small_messages_take_the_one_shot_template_between_servers():
    c = GOLD["nhr_threshold"]
    ns, nl = c["n_servers"], c["n_local"]
    for gen in (oracle.trace_hier, h.hier_emit):
        small = [o for o in gen(oracle.ALG_ALLREDUCE_NHR, ns, nl, c["oneshot_count"], oracle.F32) if o[0] == nl - 1]
        big = [o for o in gen(oracle.ALG_ALLREDUCE_NHR, ns, nl, c["sliced_count"], oracle.F32) if o[0] == nl - 1]
        seg = c["oneshot_count"] * c["unit"] // nl
        assert small and all(o[1] == 1 and o[8] == seg for o in small)            # whole segments
        assert len(small) == nl * (ns // 2)                                       # first round of the binomial tree
        assert big and all(o[1] == 1 and o[8] < seg for o in big)                 # slices of a segment
        assert len(big) >= nl * ns


@pytest.mark.parametrize("mesh", [False, True])
@pytest.mark.parametrize("alg1", LEVEL1)
def test_product_generator_equals_oracle_trace_and_passes_the_checker(alg1, mesh):
    for ns, nl in SHAPES + [(1, 2), (1, 32)]:
        if mesh and nl < 2:
            with pytest.raises(ValueError):                       # no stream to run the mesh on
                oracle.trace_hier(alg1, ns, nl, 100, oracle.F32, mesh=True)
            with pytest.raises(h.HcommError):
                h.hier_emit(alg1, ns, nl, 100, oracle.F32, mesh=True)
            continue
        for count, dt in ((100003, oracle.F32), (1000, oracle.F16), (7, oracle.I8), (0, oracle.F32),
                          (300007, oracle.I32), (8 * 70000, oracle.F32)):
            a = oracle.trace_hier(alg1, ns, nl, count, dt, mesh=mesh)
            assert a == h.hier_emit(alg1, ns, nl, count, dt, mesh=mesh), (alg1, ns, nl, count)
            assert h.hier_check(alg1, ns, nl, count, dt, mesh=mesh)[:2] == (0, 0), (alg1, ns, nl, count)
            assert h.oplist_check(a, ns * nl, Expect.ALLREDUCE, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)


@pytest.mark.parametrize("mesh", [False, True])
@pytest.mark.parametrize("alg1", LEVEL1)
def test_exact_integer_sums(alg1, mesh):
    rng = np.random.default_rng(5)
    for ns, nl in SHAPES:
        if mesh and nl < 2:
            continue
        n = ns * nl
        for count in (1, 31, 100003):
            ins = [rng.integers(-1000, 1000, count, dtype=np.int32) for _ in range(n)]
            work = [x.copy() for x in ins]
            outs = [np.full(count, -7, np.int32) for _ in range(n)]
            oracle.run_hier(alg1, ns, nl, work, outs, count, oracle.I32, oracle.SUM, mesh=mesh)
            want = np.sum(np.stack(ins).astype(np.int64), axis=0).astype(np.int32)
            for r in range(n):
                assert np.array_equal(outs[r], want), (alg1, ns, nl, count, r)


def test_rejects_bad_arguments():
    for f in (oracle.trace_hier, h.hier_emit):
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_ALLREDUCE_MESH_ONESHOT, 2, 2, 100, oracle.F32)      # not a level-1 choice of this executor
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_ALLREDUCE_RING, 8, 8, 100, oracle.F32)              # more ranks than the library simulates
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_ALLREDUCE_RING, 0, 2, 100, oracle.F32)
