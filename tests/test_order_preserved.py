"""The order-preserving reduce-scatter executor on one server (every rank plants its blocks into the peers' CCL output
buffers, every rank folds what it received along one fixed tree over rank order): the oracle's per-rank transcription
against hand-derived operation lists, fold trees and chunk tables, exact integer arithmetic, the symbolic checker and
the product's step-major generator."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))["order_preserved_reduce_scatter"]
CCL_OUT, UIN, UOUT = 1, 3, 4


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["ops_n3_fp32_count10"]["ops"]]
    assert oracle.trace_order_preserved(3, 10, 1 << 20, oracle.F32) == want
    assert h.order_preserved_emit(3, 10, 1 << 20, oracle.F32) == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_every_rank_folds_in_the_same_rank_order(op):
    for n_s, tree in GOLD["rank_tree"].items():
        n, count = int(n_s), 257
        ins = order_sensitive_inputs(n, n * count, op, seed=500 + n)
        uin = [x.copy() for x in ins]
        uout = [np.zeros(count, np.float32) for _ in range(n)]
        ccl = n * 2048
        cin = [np.zeros(1, np.float32) for _ in range(n)]
        cout = [np.zeros(ccl // 4, np.float32) for _ in range(n)]
        oracle.run_order_preserved(uin, uout, cin, cout, count, ccl, oracle.F32, op)
        for p in range(n):
            want = eval_tree(tree, [x[p * count:(p + 1) * count] for x in ins], op)
            assert np.array_equal(uout[p].view(np.uint32), want.view(np.uint32)), (n, p)
            assert np.array_equal(uin[p].view(np.uint32), ins[p].view(np.uint32))


def test_chunk_table_hand_derived():
    c = GOLD["chunks"]
    n, count, ccl = c["n"], c["count"], c["ccl_bytes"]
    for gen in (oracle.trace_order_preserved, h.order_preserved_emit):
        ops = gen(n, count, ccl, oracle.F32)
        outs = [o for o in ops if o[3] == UOUT and o[2] == 1]
        assert [o[8] for o in outs] == c["chunk_bytes"]
        assert [o[4] for o in outs] == [0, 1024, 2048]                        # consecutive in the user output
        assert [o[7] for o in outs] == [b for b in c["chunk_bytes"]]          # rank 1's slot = slot 1 of the chunk's size
        plants = [o for o in ops if o[6] == UIN and o[2] == 1 and o[5] == 0]  # what rank 0 plants into rank 1
        assert [[o[7] for o in plants]] == c["rank1_block_offsets"]
        assert [o[4] for o in plants] == [b for b in c["chunk_bytes"]]        # slot (1 + 0) mod 4


def test_product_generator_equals_oracle_trace_and_passes_the_checker():
    for n in (2, 3, 4, 5, 6, 7, 8, 12, 16, 17, 31, 32):
        for count, ccl, dt in ((1000, 1 << 20, oracle.F32), (100003, 1 << 18, oracle.F32), (7, n * 128, oracle.I8),
                               (1, n * 128, oracle.F32), (0, 4096, oracle.F32), (70001, n * 4096, oracle.F16)):
            a = oracle.trace_order_preserved(n, count, ccl, dt)
            assert a == h.order_preserved_emit(n, count, ccl, dt), (n, count, ccl)
            assert h.order_preserved_check(n, count, ccl, dt)[:2] == (0, 0), (n, count, ccl)
            assert h.oplist_check(a, n, Expect.REDUCE_SCATTER_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)
            for o in a:
                assert o[3] != UIN and o[6] != UOUT
                assert o[1] == 0 or (o[3] == CCL_OUT and o[6] == CCL_OUT and o[2] == o[5])   # reduces are local


def test_exact_integer_sums_and_chunking():
    rng = np.random.default_rng(3)
    for n in (2, 3, 4, 5, 6, 7, 8, 12, 16, 32):
        for count, ccl in ((1000, 1 << 20), (100003, 1 << 18), (7, n * 128), (1, n * 128)):
            ins = [rng.integers(-1000, 1000, n * count, dtype=np.int32) for _ in range(n)]
            uin = [x.copy() for x in ins]
            uout = [np.full(count, -7, np.int32) for _ in range(n)]
            cin = [np.full(1, -3, np.int32) for _ in range(n)]
            cout = [np.full(ccl // 4 + 1, -5, np.int32) for _ in range(n)]
            oracle.run_order_preserved(uin, uout, cin, cout, count, ccl, oracle.I32, oracle.SUM)
            for r in range(n):
                want = np.sum(np.stack([x[r * count:(r + 1) * count] for x in ins]).astype(np.int64), axis=0).astype(np.int32)
                assert np.array_equal(uout[r], want), (n, count, ccl, r)
                assert cout[r][-1] == -5 and cin[r][0] == -3


def test_rejects_bad_arguments():
    for f in (oracle.trace_order_preserved, h.order_preserved_emit):
        with pytest.raises((ValueError, h.HcommError)):
            f(1, 100, 4096, oracle.F32)                  # a single rank per module needs the inter-module stage
        with pytest.raises((ValueError, h.HcommError)):
            f(4, 100, 500, oracle.F32)                   # no 128-byte slot per rank fits the CCL buffer
        with pytest.raises((ValueError, h.HcommError)):
            f(33, 100, 1 << 20, oracle.F32)


# ---- the executor's branch for small messages: ReduceScatterHDStage on 4 or 8 ranks -----------------------------------

SMALL = GOLD["small_message_branch"]


def xor_leaves(tree, p):
    return tree ^ p if isinstance(tree, int) else [xor_leaves(tree[0], p), xor_leaves(tree[1], p)]


def test_small_branch_operation_list_hand_derived():
    want = [tuple(o) for o in SMALL["ops_n4_fp32_count4"]]
    assert oracle.trace_order_preserved_small(4, 4, 1 << 20, oracle.F32) == want
    assert h.order_preserved_small_emit(4, 4, 1 << 20, oracle.F32) == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_small_branch_folds_along_the_rank_order_tree_seen_from_each_rank(op):
    for n in (4, 8):
        count = 1000
        ins = order_sensitive_inputs(n, n * count, op, seed=1300 + n)
        uin = [x.copy() for x in ins]
        uout = [np.zeros(count, np.float32) for _ in range(n)]
        ccl = 1 << 16
        cin = [np.zeros(1, np.float32) for _ in range(n)]
        cout = [np.zeros(ccl // 4, np.float32) for _ in range(n)]
        oracle.run_order_preserved_small(uin, uout, cin, cout, count, ccl, oracle.F32, op)
        for p in range(n):
            want = eval_tree(xor_leaves(GOLD["rank_tree"][str(n)], p), [x[p * count:(p + 1) * count] for x in ins], op)
            assert np.array_equal(uout[p].view(np.uint32), want.view(np.uint32)), (n, p)
            assert np.array_equal(uin[p].view(np.uint32), ins[p].view(np.uint32))


def test_small_branch_product_equals_oracle_and_passes_the_checker():
    for n in (4, 8):
        for count, dt in ((1, oracle.F32), (4, oracle.F32), (7, oracle.I8), (8192, oracle.F32), (16384, oracle.F16),
                          (0, oracle.F32), (32768, oracle.I8), (333, oracle.I16)):
            a = oracle.trace_order_preserved_small(n, count, 1 << 20, dt)
            assert a == h.order_preserved_small_emit(n, count, 1 << 20, dt), (n, count)
            assert h.order_preserved_small_check(n, count, 1 << 20, dt)[:2] == (0, 0), (n, count)
            assert h.oplist_check(a, n, Expect.REDUCE_SCATTER_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)
            assert len(a) == (0 if count == 0 else n * (2 + n.bit_length() - 1))
            for o in a:
                assert o[3] != UIN and o[6] != UOUT and o[4] + o[8] <= n // 2 * count * h.DTYPE_SIZE[dt] or o[3] == UOUT


def test_small_branch_exact_integer_sums():
    rng = np.random.default_rng(8)
    for n in (4, 8):
        for count in (1, 7, 100, 8192):
            ins = [rng.integers(-1000, 1000, n * count, dtype=np.int32) for _ in range(n)]
            uin = [x.copy() for x in ins]
            uout = [np.full(count, -7, np.int32) for _ in range(n)]
            ccl = n * 32768
            cin = [np.full(1, -3, np.int32) for _ in range(n)]
            cout = [np.full(ccl // 4 + 1, -5, np.int32) for _ in range(n)]
            oracle.run_order_preserved_small(uin, uout, cin, cout, count, ccl, oracle.I32, oracle.SUM)
            for r in range(n):
                want = np.sum(np.stack([x[r * count:(r + 1) * count] for x in ins]).astype(np.int64), axis=0).astype(np.int32)
                assert np.array_equal(uout[r], want), (n, count, r)
                assert cout[r][-1] == -5 and np.array_equal(uin[r], ins[r])
                assert np.all(cout[r][n // 2 * count:] == -5)                 # only the first half-message is used


def test_small_branch_rejects_what_the_executor_does_not_route_to_it():
    for f in (oracle.trace_order_preserved_small, h.order_preserved_small_emit):
        for args in ((2, 100, 1 << 20, oracle.F32), (5, 100, 1 << 20, oracle.F32), (16, 100, 1 << 20, oracle.F32),
                     (8, 8193, 1 << 20, oracle.F32),          # more than 32 KiB per rank
                     (8, 1000, 8 * 3968, oracle.F32)):        # the loop would cut the message into chunks
            with pytest.raises((ValueError, h.HcommError)):
                f(*args)
