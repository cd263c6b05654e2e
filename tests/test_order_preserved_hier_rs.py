"""The order-preserving reduce-scatter executor over two communicator levels (plant + fold in device order inside every
server with an all-to-all offset of 1, plant + fold in server order between the servers, own block to the user output):
the oracle's per-rank transcription against a hand-derived operation list and hand-composed reduction trees, exact
integer arithmetic, layout invariants, the symbolic checker and the product's step-major generator."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs
from test_order_preserved_hier_ar import SHAPES, SINGLE, TREES1, two_level_tree

_G = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))
GOLD = _G["order_preserved_hier_reduce_scatter"]
TREES2 = _G["order_preserved_hier_allreduce"]["trees"]
CCL_OUT, UIN, UOUT = 1, 3, 4


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["ops_2x2_fp32_count10"]["ops"]]
    assert oracle.trace_order_preserved_rs2(2, 2, 10, 1 << 20, oracle.F32) == want
    assert h.order_preserved_hier_rs_emit(2, 2, 10, 1 << 20, oracle.F32) == want


def test_operation_list_hand_derived_one_device_per_module():
    want = [tuple(o) for o in GOLD["ops_3x1_fp32_count10"]["ops"]]
    assert oracle.trace_order_preserved_rs2(3, 1, 10, 1 << 20, oracle.F32) == want
    assert h.order_preserved_hier_rs_emit(3, 1, 10, 1 << 20, oracle.F32) == want


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_every_block_is_folded_devices_first_then_servers_in_rank_order(op):
    for m, l in ((2, 2), (2, 3), (3, 2), (2, 4), (4, 2), (3, 3), (2, 8), (4, 4), (3, 5), (5, 6), (2, 1), (3, 1), (5, 1), (8, 1)):
        n, count = m * l, 700
        ins = order_sensitive_inputs(n, n * count, op, seed=1100 + n)
        uin = [x.copy() for x in ins]
        uout = [np.zeros(count, np.float32) for _ in range(n)]
        ccl = n * 1024                                               # three chunks: 256, 256, 188 elements
        cin = [np.zeros(ccl // 4, np.float32) for _ in range(n)]
        cout = [np.zeros(ccl // 4, np.float32) for _ in range(n)]
        oracle.run_order_preserved_rs2(m, l, uin, uout, cin, cout, count, ccl, oracle.F32, op)
        tree = TREES1[str(m)] if l == 1 else TREES2.get("%dx%d" % (m, l)) or two_level_tree(m, l)
        for p in range(n):
            want = eval_tree(tree, [x[p * count:(p + 1) * count] for x in ins], op)
            assert np.array_equal(uout[p].view(np.uint32), want.view(np.uint32)), (m, l, p)
            assert np.array_equal(uin[p].view(np.uint32), ins[p].view(np.uint32))


def test_layout_invariants():
    for m, l in SHAPES:
        n, count, dt, unit = m * l, 10003, oracle.F16, 2
        ccl = n * 4096
        ops = oracle.trace_order_preserved_rs2(m, l, count, ccl, dt)
        s0, s1 = max(1, (l - 1).bit_length()), max(1, (m - 1).bit_length())
        per_chunk = 3 + s0 + s1
        max_count = ccl // n // 128 * 128 // unit
        assert max(o[0] for o in ops) + 1 == per_chunk * -(-count // max_count)
        for step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes in ops:
            k, chunk = step % per_chunk, step // per_chunk
            c = min(max_count, count - chunk * max_count) * unit
            srv, dev = divmod(rank, l)
            assert nbytes == c and 0 not in (dbuf, sbuf)                     # no CCL input buffer, no borrowed place
            if kind == 1:
                assert rank == srank and dbuf == sbuf == CCL_OUT
            if k == 0:
                b = (soff - chunk * max_count * unit) // (count * unit)
                assert sbuf == UIN and srank // l == srv and b % l == dev
                assert (dbuf, doff) == (CCL_OUT, (b // l * l + (1 + srank % l + dev) % l) * c)
            if k == 1 + s0:
                assert kind == 0 and srank % l == dev
                assert (dbuf, doff) == (CCL_OUT, (dev + (srank // l + srv) % m * l) * c)
                assert (sbuf, soff) == (CCL_OUT, ((1 + dev) % l + srv * l) * c)
            if k == per_chunk - 1:
                assert (dbuf, doff, sbuf, soff) == (UOUT, chunk * max_count * unit, CCL_OUT, rank * c)


def test_product_generator_equals_oracle_trace_and_passes_the_checker():
    for m, l in SHAPES + SINGLE:
        n = m * l
        for count, ccl, dt in ((10, 1 << 20, oracle.F32), (1000, 1 << 20, oracle.F32), (100003, 1 << 18, oracle.F16),
                               (7, n * 128, oracle.I8), (1, n * 128, oracle.F32), (0, 4096, oracle.F32)):
            a = oracle.trace_order_preserved_rs2(m, l, count, ccl, dt)
            assert a == h.order_preserved_hier_rs_emit(m, l, count, ccl, dt), (m, l, count, ccl)
            assert h.order_preserved_hier_rs_check(m, l, count, ccl, dt)[:2] == (0, 0), (m, l, count, ccl)
            assert h.oplist_check(a, n, Expect.REDUCE_SCATTER_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)


def test_exact_integer_sums_and_chunking():
    rng = np.random.default_rng(6)
    for m, l in SHAPES + SINGLE:
        n = m * l
        for count, ccl in ((1000, 1 << 20), (10003, 1 << 16), (7, n * 128), (1, n * 128)):
            ins = [rng.integers(-1000, 1000, n * count, dtype=np.int32) for _ in range(n)]
            uin = [x.copy() for x in ins]
            uout = [np.full(count, -7, np.int32) for _ in range(n)]
            cin = [np.full(ccl // 4 + 1, -3, np.int32) for _ in range(n)]
            cout = [np.full(ccl // 4 + 1, -5, np.int32) for _ in range(n)]
            oracle.run_order_preserved_rs2(m, l, uin, uout, cin, cout, count, ccl, oracle.I32, oracle.SUM)
            for r in range(n):
                want = np.sum(np.stack([x[r * count:(r + 1) * count] for x in ins]).astype(np.int64), axis=0).astype(np.int32)
                assert np.array_equal(uout[r], want), (m, l, count, ccl, r)
                assert cout[r][-1] == -5 and cin[r][-1] == -3
                assert l == 1 or np.all(cin[r] == -3)                  # only one device per module stages there
                assert np.array_equal(uin[r], ins[r])


def test_rejects_bad_arguments():
    for f in (oracle.trace_order_preserved_rs2, h.order_preserved_hier_rs_emit):
        for args in ((1, 8, 100, 4096, oracle.F32),            # one module: the single-server executor
                     (8, 0, 100, 4096, oracle.F32),
                     (2, 2, 100, 500, oracle.F32),             # no 128-byte block per rank fits the CCL buffer
                     (3, 11, 100, 1 << 20, oracle.F32)):       # more than 32 ranks
            with pytest.raises((ValueError, h.HcommError)):
                f(*args)
