"""The order-preserving allreduce executor on one server (plant with one slot borrowed from the CCL input buffer, fold
in rank order, mesh all-gather inside the CCL output buffers, chunk to the user output): the oracle's per-rank
transcription against hand-derived operation lists, fold trees and chunk tables, exact integer arithmetic, the
symbolic checker and the product's step-major generator."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs

_G = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))
GOLD = _G["order_preserved_allreduce"]
TREES = _G["order_preserved_reduce_scatter"]["rank_tree"]
CCL_IN, CCL_OUT, UIN, UOUT = 0, 1, 3, 4


def blocks(cur_bytes, n, unit):
    """Block stride and block sizes of one chunk, from the definition (not from either generator)."""
    elems = cur_bytes // unit
    stride = -(-(-(-elems // n) * unit) // 128) * 128
    return stride, [max(0, min(stride, cur_bytes - d * stride)) for d in range(n)]


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["ops_n3_fp32_count100"]["ops"]]
    assert oracle.trace_order_preserved_ar(3, 100, 1 << 20, oracle.F32) == want
    assert h.order_preserved_ar_emit(3, 100, 1 << 20, oracle.F32) == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_every_element_is_folded_in_the_same_rank_order(op):
    for n_s, tree in TREES.items():
        n, count = int(n_s), 2500
        ins = order_sensitive_inputs(n, count, op, seed=700 + n)
        uin = [x.copy() for x in ins]
        uout = [np.zeros(count, np.float32) for _ in range(n)]
        ccl = 4096                                                   # three chunks: 1024, 1024, 452 elements
        cin = [np.zeros(ccl // 4, np.float32) for _ in range(n)]
        cout = [np.zeros(ccl // 4, np.float32) for _ in range(n)]
        oracle.run_order_preserved_ar(uin, uout, cin, cout, count, ccl, oracle.F32, op)
        want = eval_tree(tree, ins, op)
        for p in range(n):
            assert np.array_equal(uout[p].view(np.uint32), want.view(np.uint32)), (n, p)
            assert np.array_equal(uin[p].view(np.uint32), ins[p].view(np.uint32))


def test_chunk_table_hand_derived():
    c = GOLD["chunks"]
    n, count, ccl = c["n"], c["count"], c["ccl_bytes"]
    for gen in (oracle.trace_order_preserved_ar, h.order_preserved_ar_emit):
        ops = gen(n, count, ccl, oracle.F32)
        assert max(o[0] for o in ops) + 1 == c["steps"]
        outs = [o for o in ops if o[3] == UOUT and o[2] == 1]
        assert [o[8] for o in outs] == c["chunk_bytes"]
        assert [o[4] for o in outs] == [0, 1024, 2048] and all(o[7] == 0 and o[6] == CCL_OUT for o in outs)
        for k, (sizes, stride) in enumerate(zip(c["block_bytes"], c["block_stride"])):
            assert blocks(c["chunk_bytes"][k], n, 4) == (stride, sizes)
            plants = [o for o in ops if o[0] == 5 * k and o[5] == 0]          # what rank 0 plants in chunk k
            assert [o[8] for o in plants] == [s for s in sizes if s]
            assert [o[7] for o in plants] == [1024 * k + d * stride for d in range(n) if sizes[d]]
            # rank 0's contribution: slot p of rank p, the borrowed slot on rank 3 - 0 = 3?  no: slot N-1 is rank 3's own
            assert [(o[2], o[3], o[4]) for o in plants] == [(d, CCL_OUT, d * stride) for d in range(n) if sizes[d]]
            gathers = [o for o in ops if o[0] == 5 * k + 3 and o[2] == 1]
            assert [(o[5], o[4], o[7], o[8]) for o in gathers] == [
                (s, s * stride, s * stride, sizes[s]) for s in (0, 3, 2) if sizes[s]]


def test_borrowed_slot_and_layout_invariants():
    for n in (2, 3, 4, 5, 8, 13, 32):
        for count, ccl, dt in ((1000, 1 << 20, oracle.F32), (100003, 1 << 16, oracle.F16), (n, 4096, oracle.I8)):
            unit = h.DTYPE_SIZE[dt]
            ops = oracle.trace_order_preserved_ar(n, count, ccl, dt)
            steps = 3 + max(1, (n - 1).bit_length())
            left, k = count * unit, 0
            while left:
                cur = min(left, ccl // unit * unit)
                stride, sizes = blocks(cur, n, unit)
                base = k * steps
                chunk = [o for o in ops if base <= o[0] < base + steps]
                for o in chunk:
                    for rank, buf, off in ((o[2], o[3], o[4]), (o[5], o[6], o[7])):
                        if buf == CCL_IN:                      # only the borrowed slot: rank p < N-1, at p * stride
                            assert rank != n - 1 and off == rank * stride and o[8] == sizes[rank]
                        if buf in (CCL_IN, CCL_OUT):
                            assert off % stride == 0 and off + o[8] <= ccl
                # slot (p + q) mod N of rank p holds rank q's block p; slot N-1 is borrowed unless p is the last rank
                for o in chunk:
                    if o[0] == base:
                        p, q = o[2], o[5]
                        assert o[6] == UIN and o[7] == k * (ccl // unit * unit) + p * stride and o[8] == sizes[p]
                        slot = (p + q) % n
                        assert (o[3], o[4]) == ((CCL_IN, p * stride) if slot == n - 1 and p != n - 1 else (CCL_OUT, slot * stride))
                left -= cur
                k += 1


def test_product_generator_equals_oracle_trace_and_passes_the_checker():
    refused = 0
    for n in (2, 3, 4, 5, 6, 7, 8, 12, 16, 17, 31, 32):
        for count, ccl, dt in ((1000, 1 << 20, oracle.F32), (100003, 1 << 18, oracle.F32), (7, 4096, oracle.I8),
                               (1, 4096, oracle.F32), (0, 4096, oracle.F32), (70001, 8192, oracle.F16),
                               (n * 32, n * 128, oracle.F32), (n * 32 + 1, n * 128 + 128, oracle.F32)):
            try:
                a = oracle.trace_order_preserved_ar(n, count, ccl, dt)
            except ValueError:                                        # the rounded-up slots do not fit: both refuse
                with pytest.raises(h.HcommError):
                    h.order_preserved_ar_emit(n, count, ccl, dt)
                refused += 1
                continue
            assert a == h.order_preserved_ar_emit(n, count, ccl, dt), (n, count, ccl)
            assert h.order_preserved_ar_check(n, count, ccl, dt)[:2] == (0, 0), (n, count, ccl)
            assert h.oplist_check(a, n, Expect.ALLREDUCE_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)
            for o in a:
                assert o[3] != UIN and o[6] != UOUT
                assert o[1] == 0 or o[2] == o[5]                     # reduces are local
    assert 0 < refused <= 16                                         # tiny buffers only


def test_exact_integer_sums_and_chunking():
    rng = np.random.default_rng(4)
    for n in (2, 3, 4, 5, 6, 7, 8, 12, 16, 32):
        for count, ccl in ((1000, 1 << 20), (100003, 1 << 18), (7, 4096), (1, 4096), (n * 32, n * 128)):
            ins = [rng.integers(-1000, 1000, count, dtype=np.int32) for _ in range(n)]
            uin = [x.copy() for x in ins]
            uout = [np.full(count, -7, np.int32) for _ in range(n)]
            cin = [np.full(ccl // 4 + 1, -3, np.int32) for _ in range(n)]
            cout = [np.full(ccl // 4 + 1, -5, np.int32) for _ in range(n)]
            oracle.run_order_preserved_ar(uin, uout, cin, cout, count, ccl, oracle.I32, oracle.SUM)
            want = np.sum(np.stack(ins).astype(np.int64), axis=0).astype(np.int32)
            for r in range(n):
                assert np.array_equal(uout[r], want), (n, count, ccl, r)
                assert cout[r][-1] == -5 and cin[r][-1] == -3
                assert np.array_equal(uin[r], ins[r])


def test_rejects_bad_arguments():
    for f in (oracle.trace_order_preserved_ar, h.order_preserved_ar_emit):
        with pytest.raises((ValueError, h.HcommError)):
            f(1, 100, 4096, oracle.F32)                  # a single rank per module needs the inter-module stage
        with pytest.raises((ValueError, h.HcommError)):
            f(4, 100, 3, oracle.F32)                     # not one element fits the CCL buffer
        with pytest.raises((ValueError, h.HcommError)):
            f(8, 16, 16, oracle.I8)                      # the 128-byte slots of a 16-byte chunk reach past 16 bytes
        with pytest.raises((ValueError, h.HcommError)):
            f(33, 100, 1 << 20, oracle.F32)


# ---- the single-launch lowering of both order-preserving executors --------------------------------------------------

def kernel_tree(n):
    """The tree the fold kernel's rank-order mode builds: position q of K = 2^L holds rank bitrev(q) if it exists;
    level l folds position q + 2^l into position q (q a multiple of 2^(l+1)) wherever the former exists."""
    L = max(1, (n - 1).bit_length())
    K = 1 << L
    rev = lambda q: int(format(q, "0%db" % L)[::-1], 2)
    x = [rev(q) if rev(q) < n else None for q in range(K)]
    for l in range(L):
        for q in range(0, K, 2 << l):
            if x[q + (1 << l)] is not None:
                x[q] = [x[q], x[q + (1 << l)]]
    return x[0]


def test_fused_kernel_tree_is_the_executors_rank_order_tree():
    for n_s, tree in TREES.items():
        assert kernel_tree(int(n_s)) == tree, n_s


def test_fused_plan_is_one_tree_launch_on_the_user_buffers():
    base = 0x7f0000000000
    for n in (2, 3, 5, 8, 17, 32):
        uin = [base + r * (1 << 32) for r in range(n)]
        uout = [base + (64 + r) * (1 << 32) for r in range(n)]
        for all_reduce, count, dt in ((1, 100003, oracle.F32), (1, 7, oracle.I8), (0, 4096, oracle.BF16), (0, 12, oracle.F32)):
            unit = h.DTYPE_SIZE[dt]
            p = h.OrderPreservedFusedPlan(all_reduce, uin, uout, count, dt, oracle.SUM)
            try:
                launches = p.launches()
                assert [l.kind for l in launches] == [h.Kernel.TREE]
                assert launches[0].nseg == (1 if all_reduce else n)
                assert launches[0].bytes == count * unit * (1 if all_reduce else n)
                ops = (oracle.trace_order_preserved_ar if all_reduce else oracle.trace_order_preserved)(n, count, 1 << 40, dt)
                assert p.info.algorithmicBytes == sum(o[8] * (3 if o[1] else 2) for o in ops)
                # what the launch itself moves: N reads per element and N (allreduce) or 1 (reduce-scatter) writes
                assert p.info.movedBytes == launches[0].bytes * (2 * n if all_reduce else n + 1)
            finally:
                p.destroy()
        with pytest.raises(h.HcommError):
            h.OrderPreservedFusedPlan(0, uin, uout, 3, oracle.F32, oracle.SUM)      # 12-byte blocks: not 16-byte multiples
        p = h.OrderPreservedFusedPlan(1, uin, uout, 0, oracle.F32, oracle.SUM)
        assert p.launches() == []
        p.destroy()
    with pytest.raises(h.HcommError):
        h.OrderPreservedFusedPlan(1, [base], [base + 4096], 16, oracle.F32, oracle.SUM)
