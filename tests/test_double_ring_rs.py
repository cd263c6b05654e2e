"""The double-ring reduce-scatter executor on one server in op-base mode with DMA reduce (both shares of every block
reduced around two mirrored rings through the CCL input buffers, the last fold landing in the user output): the oracle's
transcription in ring-position space against a hand-derived operation list, reduction trees and chunk table, exact
integer arithmetic, the symbolic checker and the product's generator, which is written in rank space."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))["double_ring_reduce_scatter"]
CCL_IN, UIN, UOUT = 0, 3, 4


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["rank0_ops_n3_fp32_count64"]["ops"]]
    for gen in (oracle.trace_dbring_rs, h.dbring_rs_emit):
        assert [o for o in gen(3, 64, 1 << 20, oracle.F32) if o[2] == 0] == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_reduction_trees_hand_derived(op):
    n, count = 4, 64
    ins = order_sensitive_inputs(n, n * count, op, seed=700)
    uin = [x.copy() for x in ins]
    uout = [np.zeros(count, np.float32) for _ in range(n)]
    cin = [np.zeros(n * count, np.float32) for _ in range(n)]
    oracle.run_dbring_rs(uin, uout, cin, count, n * count * 4, oracle.F32, op)
    for b, first, cnt, tree in GOLD["trees_n4_count64"]["pieces"]:
        want = eval_tree(tree, [x[b * count + first:b * count + first + cnt] for x in ins], op)
        assert np.array_equal(uout[b][first:first + cnt].view(np.uint32), want.view(np.uint32)), (b, first)
    for r in range(n):
        assert np.array_equal(uin[r].view(np.uint32), ins[r].view(np.uint32))


def test_chunk_table_hand_derived():
    c = GOLD["chunks"]
    for gen in (oracle.trace_dbring_rs, h.dbring_rs_emit):
        ops = gen(c["n"], c["count"], c["ccl_bytes"], oracle.F32)
        last = [o for o in ops if o[1] == 1 and o[3] == UOUT and o[2] == 1]           # rank 1's closing folds
        assert [[last[2 * k][8], last[2 * k + 1][8]] for k in range(3)] == c["shares"]
        assert [last[2 * k][4] for k in range(3)] == [0, 1024, 2048]                  # consecutive in the user output
        assert [last[2 * k][8] + last[2 * k + 1][8] for k in range(3)] == c["chunk_bytes"]


def test_product_generator_equals_oracle_trace_and_passes_the_checker():
    for n in (3, 4, 5, 7, 8, 12, 16, 17, 31, 32):
        for count, ccl, dt in ((1000, 1 << 20, oracle.F32), (10003, 1 << 17, oracle.F32), (7, n * 128, oracle.I8),
                               (1, n * 128, oracle.F32), (0, 4096, oracle.F32), (300, n * 256, oracle.F16)):
            a = oracle.trace_dbring_rs(n, count, ccl, dt)
            assert a == h.dbring_rs_emit(n, count, ccl, dt), (n, count, ccl)
            assert h.dbring_rs_check(n, count, ccl, dt)[:2] == (0, 0), (n, count, ccl)
            assert h.oplist_check(a, n, Expect.REDUCE_SCATTER_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)
            for o in a:
                assert o[3] != UIN and o[6] != UOUT                       # user input only read, user output only written
                assert o[1] == 0 or o[6] == CCL_IN                        # every fold reads a neighbour's CCL input
                if o[3] == UOUT or o[6] == UIN:
                    assert o[2] == o[5] or o[1] == 1                      # user memory is the rank's own


def test_exact_integer_sums_and_chunking():
    rng = np.random.default_rng(11)
    for n in (3, 4, 5, 7, 8, 16, 32):
        for count, ccl in ((1000, 1 << 20), (10003, 1 << 17), (7, n * 128), (1, n * 128), (300, n * 256)):
            ins = [rng.integers(-1000, 1000, n * count, dtype=np.int32) for _ in range(n)]
            uin = [x.copy() for x in ins]
            uout = [np.full(count, -7, np.int32) for _ in range(n)]
            cin = [np.full(ccl // 4 + 1, -3, np.int32) for _ in range(n)]
            oracle.run_dbring_rs(uin, uout, cin, count, ccl, oracle.I32, oracle.SUM)
            for r in range(n):
                want = np.sum(np.stack([x[r * count:(r + 1) * count] for x in ins]).astype(np.int64), axis=0).astype(np.int32)
                assert np.array_equal(uout[r], want), (n, count, ccl, r)
                assert cin[r][-1] == -3


def test_rejects_bad_arguments():
    for f in (oracle.trace_dbring_rs, h.dbring_rs_emit):
        with pytest.raises((ValueError, h.HcommError)):
            f(2, 100, 4096, oracle.F32)                  # the template's two-rank first step does not hold together
        with pytest.raises((ValueError, h.HcommError)):
            f(4, 100, 500, oracle.F32)                   # no 128-byte block per rank fits the CCL buffer
        with pytest.raises((ValueError, h.HcommError)):
            f(33, 100, 1 << 20, oracle.F32)
