"""The ring and mesh reduce-scatter executors over two communicator levels in op-base mode (user input -> CCL input,
reduce-scatter between the servers over runs of blocks, reduce-scatter inside the server over the blocks of the own
run, own block -> CCL output -> user output): the oracle's per-rank transcription against hand-derived operation
lists, reduction trees and chunk tables, exact integer arithmetic, the symbolic checker and the product's generator."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))["hier_reduce_scatter"]
LEVEL1 = {oracle.ALG_RS_RING_STAGE: h.Alg.REDUCE_SCATTER_RING, oracle.ALG_RS_NHR: h.Alg.REDUCE_SCATTER_NHR,
          oracle.ALG_RS_NB: h.Alg.REDUCE_SCATTER_NB, oracle.ALG_RS_RHD: h.Alg.REDUCE_SCATTER_RHD}
SHAPES = [(1, 8), (1, 2), (1, 3), (2, 4), (3, 5), (4, 8), (2, 2), (2, 1), (1, 1), (5, 3), (1, 16), (2, 16), (8, 4),
          (6, 2), (7, 1), (17, 1), (31, 1)]
CCL_IN, CCL_OUT, UIN, UOUT = 0, 1, 3, 4


def run(alg1, ns, nl, ins, count, ccl, dt, op, mesh, npdt=np.float32):
    n = ns * nl
    uin = [x.copy() for x in ins]
    uout = [np.zeros(count, npdt) for _ in range(n)]
    cin = [np.zeros(ccl // uout[0].itemsize + 1, npdt) for _ in range(n)]
    cout = [np.zeros(ccl // uout[0].itemsize + 1, npdt) for _ in range(n)]
    oracle.run_hier_rs(alg1, ns, nl, uin, uout, cin, cout, count, ccl, dt, op, mesh=mesh)
    for r in range(n):
        assert np.array_equal(uin[r].view(np.uint8), ins[r].view(np.uint8))          # the user input is only read
    return uout


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["ops_2x2_ring_ring_fp32_count4"]["ops"]]
    assert oracle.trace_hier_rs(oracle.ALG_RS_RING_STAGE, 2, 2, 4, 1 << 20, oracle.F32) == want
    assert h.hier_rs_emit(h.Alg.REDUCE_SCATTER_RING, 2, 2, 4, 1 << 20, oracle.F32) == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_reduction_trees_hand_derived(op):
    count = 33
    ins = order_sensitive_inputs(4, 4 * count, op, seed=600)
    out = run(oracle.ALG_RS_RING_STAGE, 2, 2, ins, count, 1 << 20, oracle.F32, op, False)
    for b_s, tree in GOLD["trees_2x2_ring_ring"].items():
        if b_s.startswith("_"):
            continue
        b = int(b_s)
        want = eval_tree(tree, [x[b * count:(b + 1) * count] for x in ins], op)
        assert np.array_equal(out[b].view(np.uint32), want.view(np.uint32)), b
    count = 96
    ins = order_sensitive_inputs(4, 4 * count, op, seed=601)
    out = run(oracle.ALG_RS_RING_STAGE, 1, 4, ins, count, 1 << 20, oracle.F32, op, True)
    for b, first, cnt, tree in GOLD["trees_1x4_mesh_count96"]["pieces"]:
        want = eval_tree(tree, [x[b * count + first:b * count + first + cnt] for x in ins], op)
        assert np.array_equal(out[b][first:first + cnt].view(np.uint32), want.view(np.uint32)), (b, first)


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_recursive_halving_doubling_between_servers_hand_derived(op):
    for n_s, trees in GOLD["trees_rhd_between_servers"].items():
        if n_s.startswith("_"):
            continue
        n, count = int(n_s), 33
        ins = order_sensitive_inputs(n, n * count, op, seed=610 + n)
        out = run(oracle.ALG_RS_RHD, n, 1, ins, count, 1 << 20, oracle.F32, op, False)
        for b_s, tree in trees.items():
            b = int(b_s)
            want = eval_tree(tree, [x[b * count:(b + 1) * count] for x in ins], op)
            assert np.array_equal(out[b].view(np.uint32), want.view(np.uint32)), (n, b)
    for f, a in ((oracle.trace, oracle.ALG_RS_RHD), (h.schedule_emit, h.Alg.REDUCE_SCATTER_RHD)):
        with pytest.raises((ValueError, h.HcommError)):      # only between the servers of the two-level reduce-scatter
            f(a, 4, 100, oracle.F32)


def test_chunk_table_hand_derived():
    c = GOLD["chunks"]
    ns, nl, count, ccl = c["n_servers"], c["n_local"], c["count"], c["ccl_bytes"]
    for gen, alg in ((oracle.trace_hier_rs, oracle.ALG_RS_RING_STAGE), (h.hier_rs_emit, h.Alg.REDUCE_SCATTER_RING)):
        ops = gen(alg, ns, nl, count, ccl, oracle.F32)
        outs = [o for o in ops if o[3] == UOUT and o[2] == 0]
        assert [o[8] for o in outs] == c["chunk_bytes"]
        assert [o[4] for o in outs] == [0, 164, 328]
        ins = [o for o in ops if o[6] == UIN and o[2] == 0]
        assert len(ins) == 3 * ns * nl                                 # block by block: no chunk takes everything
        blk4 = [o for o in ins if o[7] in c["rank0_block4_src"]]
        assert [o[7] for o in blk4] == c["rank0_block4_src"] and [o[4] for o in blk4] == c["rank0_block4_dst"]
    # a single chunk that takes everything: one copy of the whole input
    ops = oracle.trace_hier_rs(oracle.ALG_RS_RING_STAGE, ns, nl, 41, ccl, oracle.F32)
    assert [o[8] for o in ops if o[6] == UIN and o[2] == 0] == [41 * 4 * ns * nl]


@pytest.mark.parametrize("mesh", [False, True])
@pytest.mark.parametrize("alg1", sorted(LEVEL1))
def test_product_generator_equals_oracle_trace_and_passes_the_checker(alg1, mesh):
    for ns, nl in SHAPES:
        n = ns * nl
        if mesh and nl < 2:
            for f, a in ((oracle.trace_hier_rs, alg1), (h.hier_rs_emit, LEVEL1[alg1])):
                with pytest.raises((ValueError, h.HcommError)):           # no stream to run the mesh on
                    f(a, ns, nl, 100, 1 << 20, oracle.F32, mesh=True)
            continue
        for count, ccl, dt in ((1000, 1 << 20, oracle.F32), (10003, 1 << 17, oracle.F32), (7, n * 28, oracle.I8),
                               (1, n * 4, oracle.F32), (0, 4096, oracle.F32), (9001, n * 4096, oracle.F16)):
            a = oracle.trace_hier_rs(alg1, ns, nl, count, ccl, dt, mesh=mesh)
            assert a == h.hier_rs_emit(LEVEL1[alg1], ns, nl, count, ccl, dt, mesh=mesh), (alg1, ns, nl, count, ccl)
            assert h.hier_rs_check(LEVEL1[alg1], ns, nl, count, ccl, dt, mesh=mesh)[:2] == (0, 0), (alg1, ns, nl, count)
            assert h.oplist_check(a, n, Expect.REDUCE_SCATTER_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)
            for o in a:
                assert o[3] != UIN and o[6] != UOUT
                assert o[1] == 0 or (o[3] == CCL_IN and o[6] == CCL_IN)             # reduces stay in the CCL inputs


@pytest.mark.parametrize("mesh", [False, True])
@pytest.mark.parametrize("alg1", sorted(LEVEL1))
def test_exact_integer_sums_and_chunking(alg1, mesh):
    rng = np.random.default_rng(7)
    for ns, nl in SHAPES:
        if mesh and nl < 2:
            continue
        n = ns * nl
        for count, ccl in ((1000, 1 << 20), (10003, 1 << 17), (7, n * 28), (1, n * 4)):
            ins = [rng.integers(-1000, 1000, n * count, dtype=np.int32) for _ in range(n)]
            out = run(alg1, ns, nl, ins, count, ccl, oracle.I32, oracle.SUM, mesh, np.int32)
            for r in range(n):
                want = np.sum(np.stack([x[r * count:(r + 1) * count] for x in ins]).astype(np.int64), axis=0).astype(np.int32)
                assert np.array_equal(out[r], want), (alg1, mesh, ns, nl, count, ccl, r)


def test_rejects_bad_arguments():
    for f, ring, ar in ((oracle.trace_hier_rs, oracle.ALG_RS_RING_STAGE, oracle.ALG_ALLREDUCE_RING),
                        (h.hier_rs_emit, h.Alg.REDUCE_SCATTER_RING, h.Alg.ALLREDUCE_RING)):
        with pytest.raises((ValueError, h.HcommError)):
            f(ar, 2, 2, 100, 1 << 20, oracle.F32)                    # not a reduce-scatter between the servers
        with pytest.raises((ValueError, h.HcommError)):
            f(ring, 2, 2, 100, 15, oracle.F32)                       # CCL buffer smaller than one element per block
        with pytest.raises((ValueError, h.HcommError)):
            f(ring, 8, 8, 100, 1 << 20, oracle.F32)
