"""The double-ring reduce-scatter executor over several servers and super pods in op-base mode with DMA reduce (every
ring position carries one slice per server of every pod; the ring folds stay in the CCL input buffers; ring, NHR or NB
between the servers of a pod, then between the pods; the own block copied out): the oracle's transcription in
ring-position space against a hand-derived operation list, reduction trees and chunk table, exact integer arithmetic, the
symbolic checker and the product's generator, which is written in rank space."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))["double_ring_reduce_scatter_servers"]
CCL_IN, UIN, UOUT = 0, 3, 4
RING, NHR, NB = oracle.ALG_RS_RING_STAGE, oracle.ALG_RS_NHR, oracle.ALG_RS_NB
SHAPES = ((2, 3), (2, 4), (3, 3), (2, 8), (4, 8), (3, 5), (5, 4), (2, 16), (10, 3), (7, 4))


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["rank0_ops_s2_n3_fp32_count64"]["ops"]]
    for gen in (oracle.trace_dbring_rs_servers, h.dbring_hier_rs_emit):
        assert [o for o in gen(RING, 2, 3, 64, 1 << 20, oracle.F32) if o[2] == 0] == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_reduction_trees_hand_derived(op):
    n_servers, n_local, count = 2, 3, 64
    n = n_servers * n_local
    ins = order_sensitive_inputs(n, n * count, op, seed=710)
    uin = [x.copy() for x in ins]
    uout = [np.zeros(count, np.float32) for _ in range(n)]
    cin = [np.zeros(n * count, np.float32) for _ in range(n)]
    oracle.run_dbring_rs_servers(RING, n_servers, n_local, uin, uout, cin, count, n * count * 4, oracle.F32, op)
    for b, first, cnt, tree in GOLD["trees_s2_n3_count64"]["pieces"]:
        want = eval_tree(tree, [x[b * count + first:b * count + first + cnt] for x in ins], op)
        assert np.array_equal(uout[b][first:first + cnt].view(np.uint32), want.view(np.uint32)), (b, first)
    for r in range(n):
        assert np.array_equal(uin[r].view(np.uint32), ins[r].view(np.uint32))


def test_chunk_table_hand_derived():
    c = GOLD["chunks"]
    for gen in (oracle.trace_dbring_rs_servers, h.dbring_hier_rs_emit):
        ops = gen(RING, c["n_servers"], c["n_local"], c["count"], c["ccl_bytes"], oracle.F32)
        for o in c["present"]:
            assert tuple(o) in ops, o
        assert [o for o in ops if o[2] == 1 and o[3] == UOUT] == [tuple(o) for o in c["rank1_out"]]


def test_product_generator_equals_oracle_trace_and_passes_the_checker():
    for alg in (RING, NHR, NB):
        for n_servers, n_local in SHAPES:
            n = n_servers * n_local
            for count, ccl, dt in ((1000, 1 << 20, oracle.F32), (10003, 1 << 17, oracle.F32), (7, n * 128, oracle.I8),
                                   (1, n * 128, oracle.F32), (0, 4096, oracle.F32), (300, n * 256, oracle.F16)):
                a = oracle.trace_dbring_rs_servers(alg, n_servers, n_local, count, ccl, dt)
                assert a == h.dbring_hier_rs_emit(alg, n_servers, n_local, count, ccl, dt), (alg, n_servers, n_local, count, ccl)
                assert h.dbring_hier_rs_check(alg, n_servers, n_local, count, ccl, dt)[:2] == (0, 0), (alg, n_servers, n_local, count)
                assert h.oplist_check(a, n, Expect.REDUCE_SCATTER_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)
                for o in a:
                    assert o[3] != UIN and o[6] != UOUT                   # user input only read, user output only written
                    assert o[1] == 0 or (o[3] == CCL_IN and o[6] == CCL_IN)  # every fold: a peer's CCL input into the own
                    if o[1] == 1:
                        same_server = o[2] // n_local == o[5] // n_local
                        same_local = o[2] % n_local == o[5] % n_local
                        assert same_server != same_local                  # a ring neighbour, or the same device of another server
                    else:
                        assert o[2] == o[5]                               # copies stay on the rank


def test_exact_integer_sums_and_chunking():
    rng = np.random.default_rng(12)
    for alg in (RING, NHR, NB):
        for n_servers, n_local in SHAPES[:8]:
            n = n_servers * n_local
            for count, ccl in ((1000, 1 << 20), (10003, 1 << 17), (7, n * 128), (1, n * 128), (300, n * 256)):
                ins = [rng.integers(-1000, 1000, n * count, dtype=np.int32) for _ in range(n)]
                uin = [x.copy() for x in ins]
                uout = [np.full(count, -7, np.int32) for _ in range(n)]
                cin = [np.full(ccl // 4 + 1, -3, np.int32) for _ in range(n)]
                oracle.run_dbring_rs_servers(alg, n_servers, n_local, uin, uout, cin, count, ccl, oracle.I32, oracle.SUM)
                for r in range(n):
                    want = np.sum(np.stack([x[r * count:(r + 1) * count] for x in ins]).astype(np.int64), axis=0).astype(np.int32)
                    assert np.array_equal(uout[r], want), (alg, n_servers, n_local, count, ccl, r)
                    assert cin[r][-1] == -3
                    assert np.array_equal(uin[r], ins[r])


def test_level1_order_differs_between_the_algorithms():
    """Four servers: ring, NHR and NB fold the servers' partial results in different orders, which floating-point sums
    show; all of them agree on integers (above)."""
    n_servers, n_local, count = 4, 3, 96
    n = n_servers * n_local
    ins = order_sensitive_inputs(n, n * count, oracle.SUM, seed=711)
    res = {}
    for alg in (RING, NHR, NB):
        uout = [np.zeros(count, np.float32) for _ in range(n)]
        cin = [np.zeros(n * count, np.float32) for _ in range(n)]
        oracle.run_dbring_rs_servers(alg, n_servers, n_local, [x.copy() for x in ins], uout, cin, count, n * count * 4, oracle.F32, oracle.SUM)
        res[alg] = np.concatenate(uout).view(np.uint32)
    assert not np.array_equal(res[RING], res[NHR])


def test_pods_operation_list_and_trees_hand_derived():
    gold = GOLD["pods"]
    for gen in (oracle.trace_dbring_rs_servers, h.dbring_hier_rs_emit):
        ops = gen(RING, 2, 3, 64, 1 << 20, oracle.F32, n_pods=2, alg2=RING)
        assert [o for o in ops if o[2] == 0 and o[0] >= 3] == [tuple(o) for o in gold["rank0_ops_from_step3"]]
        assert [o for o in ops if o[2] == 0 and o[0] == 0 and o[4] % 256 == 0] == [tuple(o) for o in gold["rank0_step0_ring0"]]
    n, count = 12, 64
    for op in (oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN):
        ins = order_sensitive_inputs(n, n * count, op, seed=712)
        uout = [np.zeros(count, np.float32) for _ in range(n)]
        cin = [np.zeros(n * count, np.float32) for _ in range(n)]
        oracle.run_dbring_rs_servers(RING, 2, 3, [x.copy() for x in ins], uout, cin, count, n * count * 4, oracle.F32, op,
                                     n_pods=2, alg2=RING)
        for b, first, cnt, tree in gold["trees"]:
            want = eval_tree(tree, [x[b * count + first:b * count + first + cnt] for x in ins], op)
            assert np.array_equal(uout[b][first:first + cnt].view(np.uint32), want.view(np.uint32)), (op, b, first)


def test_pods_product_generator_equals_oracle_trace_and_passes_the_checker():
    for a1 in (RING, NHR, NB):
        for a2 in (RING, NHR, NB):
            for n_pods, n_servers, n_local in ((2, 1, 3), (2, 2, 3), (2, 2, 8), (3, 2, 4), (2, 3, 5), (4, 2, 4), (5, 1, 6), (3, 3, 3), (8, 1, 4)):
                n = n_pods * n_servers * n_local
                for count, ccl, dt in ((1000, 1 << 20, oracle.F32), (10003, 1 << 17, oracle.F32), (7, n * 128, oracle.I8),
                                       (300, n * 256, oracle.F16)):
                    a = oracle.trace_dbring_rs_servers(a1, n_servers, n_local, count, ccl, dt, n_pods=n_pods, alg2=a2)
                    assert a == h.dbring_hier_rs_emit(a1, n_servers, n_local, count, ccl, dt, n_pods=n_pods, alg2=a2)
                    assert h.dbring_hier_rs_check(a1, n_servers, n_local, count, ccl, dt, n_pods=n_pods, alg2=a2)[:2] == (0, 0)
                    assert h.oplist_check(a, n, Expect.REDUCE_SCATTER_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)


def test_pods_exact_integer_sums():
    rng = np.random.default_rng(13)
    for a1, a2, n_pods, n_servers, n_local in ((RING, NHR, 2, 2, 3), (NHR, NB, 3, 2, 4), (NB, RING, 2, 3, 5), (RING, RING, 4, 1, 8),
                                               (NHR, NHR, 2, 2, 8)):
        n = n_pods * n_servers * n_local
        for count, ccl in ((1000, 1 << 20), (10003, 1 << 17), (7, n * 128)):
            ins = [rng.integers(-1000, 1000, n * count, dtype=np.int32) for _ in range(n)]
            uin = [x.copy() for x in ins]
            uout = [np.full(count, -7, np.int32) for _ in range(n)]
            cin = [np.full(ccl // 4 + 1, -3, np.int32) for _ in range(n)]
            oracle.run_dbring_rs_servers(a1, n_servers, n_local, uin, uout, cin, count, ccl, oracle.I32, oracle.SUM,
                                         n_pods=n_pods, alg2=a2)
            for r in range(n):
                want = np.sum(np.stack([x[r * count:(r + 1) * count] for x in ins]).astype(np.int64), axis=0).astype(np.int32)
                assert np.array_equal(uout[r], want), (a1, a2, n_pods, n_servers, n_local, count, ccl, r)
                assert cin[r][-1] == -3


def test_rejects_bad_arguments():
    for f in (oracle.trace_dbring_rs_servers, h.dbring_hier_rs_emit):
        with pytest.raises((ValueError, h.HcommError)):
            f(RING, 1, 4, 100, 1 << 20, oracle.F32)      # one server in one pod: the executor's other branch (user output written by the ring)
        with pytest.raises((ValueError, h.HcommError)):
            f(RING, 2, 2, 100, 1 << 20, oracle.F32)      # the template's two-rank first step does not hold together
        with pytest.raises((ValueError, h.HcommError)):
            f(RING, 2, 4, 100, 1000, oracle.F32)         # no 128-byte block per rank fits the CCL buffer
        with pytest.raises((ValueError, h.HcommError)):
            f(RING, 3, 11, 100, 1 << 20, oracle.F32)     # 33 ranks
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_RS_RHD, 2, 4, 100, 1 << 20, oracle.F32)  # halving-doubling is not among this executor's level-1 choices
        with pytest.raises((ValueError, h.HcommError)):
            f(RING, 2, 4, 100, 1 << 20, oracle.F32, n_pods=5)     # 40 ranks
