"""The double-ring allreduce executor in op-base mode with DMA reduce (user buffers read and written directly, the two
shares of every segment reduced and gathered around two mirrored rings, the CCL input filled slice by slice): the
oracle's transcription in ring-position space against hand-derived slice tables, operation lists and reduction trees,
against exact integer arithmetic, against the symbolic checker and against the product's generator, which is written
in rank space."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))["double_ring_allreduce"]
LEVEL1 = [oracle.ALG_ALLREDUCE_RING, oracle.ALG_ALLREDUCE_NHR, oracle.ALG_ALLREDUCE_NB]
SHAPES = [(1, 8), (1, 1), (1, 2), (1, 3), (2, 4), (3, 5), (4, 8), (2, 2), (2, 1), (1, 16), (1, 32)]
CCL_IN, CCL_OUT, UIN, UOUT = 0, 1, 3, 4


def test_slice_tables_hand_derived():
    c = GOLD["slices_n4_fp32_count1000"]
    slices, order = oracle.dbring_slices(1000, oracle.F32, 4)
    assert order == c["order"]
    assert slices == [[tuple(x) for x in ring] for ring in c["slices"]]
    for n in range(1, 33):                     # the shares tile the buffer; share 0 is 128-byte aligned in size
        for count in (0, 1, 31, 100003):
            slices, order = oracle.dbring_slices(count, oracle.I8, n)
            seg = oracle.slices_ring(count, 1, n)
            assert order[0] == list(range(n)) and order[1] == [0] + list(range(n - 1, 0, -1))
            for pos in range(n):
                a, b = slices[0][order[0].index(pos)], slices[1][order[1].index(pos)]
                assert a[0] == seg[pos][0] and a[1] + b[1] == seg[pos][1]
                assert b[0] == (a[0] + a[1] if b[1] else seg[pos][0])      # an empty share sits at the segment's start
                assert a[1] % 128 == 0 or b[1] == 0
                assert b[1] <= a[1]


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["rank0_ops_1x3_ring_fp32_count192"]["ops"]]
    for gen in (oracle.trace_dbring, h.dbring_emit):
        got = [o for o in gen(oracle.ALG_ALLREDUCE_RING, 1, 3, 192, 1 << 20, oracle.F32) if o[2] == 0]
        assert got == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_reduction_trees_hand_derived(op):
    n, count = 4, 256
    ins = order_sensitive_inputs(n, count, op, seed=400)
    uin = [x.copy() for x in ins]
    uout = [np.zeros(count, np.float32) for _ in range(n)]
    cin = [np.zeros(count, np.float32) for _ in range(n)]
    cout = [np.zeros(count, np.float32) for _ in range(n)]
    oracle.run_dbring(oracle.ALG_ALLREDUCE_RING, 1, n, uin, uout, cin, cout, count, count * 4, oracle.F32, op)
    for first, cnt, tree in GOLD["trees_1x4_fp32_count256"]["pieces"]:
        want = eval_tree(tree, [x[first:first + cnt] for x in ins], op)
        for r in range(n):
            assert np.array_equal(uout[r][first:first + cnt].view(np.uint32), want.view(np.uint32)), (first, r)
    for r in range(n):
        assert np.array_equal(uin[r].view(np.uint32), ins[r].view(np.uint32))         # the user input is only read


CONFIGS = [(100003, 1 << 20, oracle.F32), (100003, 1 << 17, oracle.F32), (7, 4096, oracle.I8), (1, 4096, oracle.F32),
           (300007, 200000, oracle.I32), (0, 4096, oracle.F32), (1000, 2048, oracle.F16)]


@pytest.mark.parametrize("alg1", LEVEL1)
def test_product_generator_equals_oracle_trace_and_passes_the_checker(alg1):
    for ns, nl in SHAPES:
        for count, ccl, dt in CONFIGS:
            a = oracle.trace_dbring(alg1, ns, nl, count, ccl, dt)
            assert a == h.dbring_emit(alg1, ns, nl, count, ccl, dt), (alg1, ns, nl, count, ccl)
            assert h.dbring_check(alg1, ns, nl, count, ccl, dt)[:2] == (0, 0), (alg1, ns, nl, count, ccl)
            assert h.oplist_check(a, ns * nl, Expect.ALLREDUCE_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)
            for o in a:                                      # the user input is only read, the user output only written
                assert o[3] != UIN and o[6] != UOUT
                assert o[1] == 0 or (o[3] == CCL_IN and o[6] == CCL_IN)        # reduces stay in the CCL input buffers
                if o[6] == UIN or o[3] == UOUT:
                    assert o[2] == o[5] or (o[3] == UOUT and o[6] == CCL_OUT)  # user memory is the rank's own


@pytest.mark.parametrize("alg1", LEVEL1)
def test_exact_integer_sums_and_chunking(alg1):
    rng = np.random.default_rng(9)
    for ns, nl in SHAPES:
        n = ns * nl
        for count, ccl in ((100003, 1 << 20), (100003, 1 << 17), (7, 4096), (1, 4096), (300007, 200000)):
            ins = [rng.integers(-1000, 1000, count, dtype=np.int32) for _ in range(n)]
            uin = [x.copy() for x in ins]
            uout = [np.full(count, -7, np.int32) for _ in range(n)]
            cin = [np.full(ccl // 4 + 1, -3, np.int32) for _ in range(n)]
            cout = [np.full(ccl // 4 + 1, -5, np.int32) for _ in range(n)]
            oracle.run_dbring(alg1, ns, nl, uin, uout, cin, cout, count, ccl, oracle.I32, oracle.SUM)
            want = np.sum(np.stack(ins).astype(np.int64), axis=0).astype(np.int32)
            for r in range(n):
                assert np.array_equal(uout[r], want), (alg1, ns, nl, count, ccl, r)
                assert np.array_equal(uin[r], ins[r])
                assert cin[r][-1] == -3 and cout[r][-1] == -5          # nothing beyond the CCL buffers


def test_moves_fewer_bytes_than_the_staged_loop():
    """What DMA reduce is for: per chunk the staged loop copies the whole message into and out of the CCL buffers on top
    of the ring's traffic; here only the slices travel."""
    n, count, ccl = 8, 1 << 20, 200 << 20
    direct = sum(o[8] * (3 if o[1] else 2) for o in oracle.trace_dbring(oracle.ALG_ALLREDUCE_RING, 1, n, count, ccl, oracle.F32))
    staged = oracle.algorithmic_bytes_opbase(oracle.ALG_ALLREDUCE_RING, n, count, ccl, oracle.F32)
    assert direct < staged
    s = count * 4
    assert direct == n * (2 * s + 3 * (n - 1) * s // n + 2 * s // n + 2 * (n - 1) * s // n + 2 * (n - 1) * s // n)


def test_rejects_bad_arguments():
    for f in (oracle.trace_dbring, h.dbring_emit):
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_ALLREDUCE_RHD, 1, 4, 100, 4096, oracle.F32)         # not a level-1 choice of this executor
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_ALLREDUCE_RING, 1, 4, 100, 3, oracle.F32)           # CCL buffer smaller than one element
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_ALLREDUCE_RING, 5, 8, 100, 4096, oracle.F32)        # more ranks than the library simulates
