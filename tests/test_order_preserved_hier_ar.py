"""The order-preserving allreduce executor over two communicator levels (plant + fold in device order inside every
server with an all-to-all offset of 1, plant + fold in server order between the servers, mesh all-gather inside,
ring / NB / NHR all-gather between the servers): the oracle's per-rank transcription against a hand-derived operation
list and hand-composed reduction trees, exact integer arithmetic, layout invariants, the symbolic checker and the
product's step-major generator."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect
from test_oracle_schedules import eval_tree, order_sensitive_inputs

_G = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))
GOLD = _G["order_preserved_hier_allreduce"]
TREES1 = _G["order_preserved_reduce_scatter"]["rank_tree"]
CCL_IN, CCL_OUT, UIN, UOUT = 0, 1, 3, 4
ALGS = [oracle.ALG_ALLREDUCE_RING, oracle.ALG_ALLREDUCE_NHR, oracle.ALG_ALLREDUCE_NB]
SHAPES = [(2, 2), (2, 3), (3, 2), (2, 8), (4, 4), (3, 5), (5, 3), (4, 8), (8, 4), (2, 16), (16, 2), (7, 3)]
SINGLE = [(2, 1), (3, 1), (5, 1), (8, 1), (13, 1), (32, 1)]          # one device per module


def compose(tree, leaves):
    return leaves[tree] if isinstance(tree, int) else [compose(tree[0], leaves), compose(tree[1], leaves)]


def relabel(tree, base):
    return tree + base if isinstance(tree, int) else [relabel(tree[0], base), relabel(tree[1], base)]


def two_level_tree(m, l):
    """tree over the servers of the trees over each server's devices - both the single-server rank-order tree."""
    return compose(TREES1[str(m)], [relabel(TREES1[str(l)], s * l) for s in range(m)])


def test_operation_list_hand_derived():
    want = [tuple(o) for o in GOLD["ops_2x2_ring_fp32_count100"]["ops"]]
    assert oracle.trace_order_preserved_ar2(oracle.ALG_ALLREDUCE_RING, 2, 2, 100, 1 << 20, oracle.F32) == want
    assert h.order_preserved_hier_ar_emit(h.Alg.ALLREDUCE_RING, 2, 2, 100, 1 << 20, oracle.F32) == want


def test_operation_list_hand_derived_one_device_per_module():
    want = [tuple(o) for o in GOLD["ops_3x1_ring_fp32_count100"]["ops"]]
    assert oracle.trace_order_preserved_ar2(oracle.ALG_ALLREDUCE_RING, 3, 1, 100, 1 << 20, oracle.F32) == want
    assert h.order_preserved_hier_ar_emit(h.Alg.ALLREDUCE_RING, 3, 1, 100, 1 << 20, oracle.F32) == want


def test_hand_composed_trees_are_the_composition_of_the_single_level_trees():
    for key, tree in GOLD["trees"].items():
        if key.startswith("_"):
            continue
        m, l = (int(x) for x in key.split("x"))
        assert two_level_tree(m, l) == tree, key


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
@pytest.mark.parametrize("alg", ALGS)
def test_every_element_is_folded_devices_first_then_servers_in_rank_order(op, alg):
    for m, l in ((2, 2), (2, 3), (3, 2), (2, 4), (4, 2), (3, 3), (2, 8), (4, 4), (3, 5), (8, 2), (5, 6), (2, 1), (3, 1), (5, 1),
                 (8, 1)):
        n, count = m * l, 80000
        ins = order_sensitive_inputs(n, count, op, seed=900 + n)
        uin = [x.copy() for x in ins]
        uout = [np.zeros(count, np.float32) for _ in range(n)]
        ccl = 1 << 17                                                # three chunks: 32768, 32768, 14464 elements
        cin = [np.zeros(ccl // 4, np.float32) for _ in range(n)]
        cout = [np.zeros(ccl // 4, np.float32) for _ in range(n)]
        oracle.run_order_preserved_ar2(alg, m, l, uin, uout, cin, cout, count, ccl, oracle.F32, op)
        tree = TREES1[str(m)] if l == 1 else GOLD["trees"].get("%dx%d" % (m, l)) or two_level_tree(m, l)
        want = eval_tree(tree, ins, op)
        for p in range(n):
            assert np.array_equal(uout[p].view(np.uint32), want.view(np.uint32)), (m, l, p)
            assert np.array_equal(uin[p].view(np.uint32), ins[p].view(np.uint32))


def test_layout_invariants():
    for m, l in SHAPES:
        n = m * l
        for alg in ALGS:
            count, ccl, dt = 100003, 1 << 17, oracle.F16
            ops = oracle.trace_order_preserved_ar2(alg, m, l, count, ccl, dt)
            unit = 2
            s0, s1 = max(1, (l - 1).bit_length()), max(1, (m - 1).bit_length())
            ag1 = m - 1 if alg == oracle.ALG_ALLREDUCE_RING else s1
            per_chunk = 4 + s0 + s1 + ag1
            assert max(o[0] for o in ops) + 1 == per_chunk * -(-count * unit // ccl)
            for o in ops:
                step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes = o
                k = step % per_chunk
                cur = min(ccl, count * unit - (step // per_chunk) * ccl)
                blk = -(-(-(-(cur // unit) // n) * unit) // 128) * 128
                srv, dev = divmod(rank, l)
                if kind == 1:
                    assert rank == srank                                         # every fold is local
                if k == 0:                                                       # level-0 plants stay inside the server
                    assert sbuf == UIN and srank // l == srv and soff % blk == (step // per_chunk) * ccl % blk
                    b = (soff - (step // per_chunk) * ccl) // blk
                    assert b % l == dev                                          # block g * L + i goes to device i
                    slot = (1 + srank % l + dev) % l
                    borrowed = slot == l - 1 and not (dev == l - 1 and b // l == m - 1)
                    assert (dbuf, doff) == ((CCL_IN, b * blk) if borrowed else (CCL_OUT, (b // l * l + slot) * blk))
                if k == 1 + s0:                                                  # level-1 plants stay on the device index
                    assert srank % l == dev and kind == 0
                    slot = (srank // l + srv) % m
                    borrowed = dev == l - 1 and slot == m - 1 and srv != m - 1
                    assert (dbuf, doff) == ((CCL_IN, rank * blk) if borrowed else (CCL_OUT, (dev + slot * l) * blk))
                    assert sbuf == (CCL_IN if dev == l - 2 else CCL_OUT)
                    assert soff == (rank if dev == l - 2 else (1 + dev) % l + srv * l) * blk
                if CCL_IN in (dbuf, sbuf):
                    assert k <= 1 + s0 + s1                                      # the gathers never touch the CCL input
                for buf, off in ((dbuf, doff), (sbuf, soff)):
                    if buf in (CCL_IN, CCL_OUT):
                        assert off + nbytes <= ccl


def test_product_generator_equals_oracle_trace_and_passes_the_checker():
    refused = 0
    for m, l in SHAPES + SINGLE:
        n = m * l
        for alg in ALGS:
            for count, ccl, dt in ((100, 1 << 20, oracle.F32), (1000, 1 << 20, oracle.F32), (100003, 1 << 18, oracle.F16),
                                   (n * 32, n * 128, oracle.F32), (7, 1 << 16, oracle.I8), (0, 4096, oracle.F32),
                                   (n * 32 + 1, n * 128 + 128, oracle.F32)):
                try:
                    a = oracle.trace_order_preserved_ar2(alg, m, l, count, ccl, dt)
                except ValueError:                                    # the rounded-up slots do not fit: both refuse
                    with pytest.raises(h.HcommError):
                        h.order_preserved_hier_ar_emit(alg, m, l, count, ccl, dt)
                    refused += 1
                    continue
                assert a == h.order_preserved_hier_ar_emit(alg, m, l, count, ccl, dt), (m, l, alg, count, ccl)
                assert h.order_preserved_hier_ar_check(alg, m, l, count, ccl, dt)[:2] == (0, 0), (m, l, alg, count, ccl)
                assert h.oplist_check(a, n, Expect.ALLREDUCE_USER, count, h.DTYPE_SIZE[dt])[:2] == (0, 0)
    assert 0 < refused <= 3 * len(SHAPES + SINGLE)


def test_exact_integer_sums_and_chunking():
    rng = np.random.default_rng(5)
    for m, l in SHAPES + SINGLE:
        n = m * l
        for alg in ALGS:
            for count, ccl in ((1000, 1 << 20), (100003, 1 << 18), (n * 32, n * 128), (7, 1 << 16), (1, 1 << 16)):
                ins = [rng.integers(-1000, 1000, count, dtype=np.int32) for _ in range(n)]
                uin = [x.copy() for x in ins]
                uout = [np.full(count, -7, np.int32) for _ in range(n)]
                cin = [np.full(ccl // 4 + 1, -3, np.int32) for _ in range(n)]
                cout = [np.full(ccl // 4 + 1, -5, np.int32) for _ in range(n)]
                try:
                    oracle.run_order_preserved_ar2(alg, m, l, uin, uout, cin, cout, count, ccl, oracle.I32, oracle.SUM)
                except ValueError:                                    # (32 x 1, 128 bytes per rank): the slots do not fit
                    assert (m, l, count, ccl) == (32, 1, n * 32, n * 128)
                    continue
                want = np.sum(np.stack(ins).astype(np.int64), axis=0).astype(np.int32)
                for r in range(n):
                    assert np.array_equal(uout[r], want), (m, l, alg, count, ccl, r)
                    assert cout[r][-1] == -5 and cin[r][-1] == -3
                    assert np.array_equal(uin[r], ins[r])


def test_rejects_bad_arguments():
    R = oracle.ALG_ALLREDUCE_RING
    for f in (oracle.trace_order_preserved_ar2, h.order_preserved_hier_ar_emit):
        for args in ((R, 1, 8, 100, 4096, oracle.F32),         # one module: the single-server executor
                     (R, 8, 0, 100, 4096, oracle.F32),
                     (R, 2, 2, 100, 3, oracle.F32),            # not one element fits the CCL buffer
                     (R, 4, 8, 16, 16, oracle.I8),             # the 128-byte slots reach past 16 bytes
                     (R, 3, 11, 100, 1 << 20, oracle.F32),     # more than 32 ranks
                     (oracle.ALG_ALLREDUCE_RHD, 2, 2, 100, 1 << 20, oracle.F32)):
            with pytest.raises((ValueError, h.HcommError)):
                f(*args)


# ---- the single-launch lowering over servers x devices ---------------------------------------------------------------

def kernel_tree_two_level(m, l):
    """The tree the fold kernel builds from the leaf table the host lays out for m servers of l devices: leaf q holds
    (server bitrev(high bits), device bitrev(low bits)) where both exist; level k folds position q + 2^k into q."""
    bl, bs = (l - 1).bit_length(), (m - 1).bit_length()
    rev = lambda q, bits: int(format(q, "0%db" % bits)[::-1], 2) if bits else 0
    x = []
    for q in range(1 << (bl + bs)):
        dev, srv = rev(q & ((1 << bl) - 1), bl), rev(q >> bl, bs)
        x.append(srv * l + dev if dev < l and srv < m else None)
    for k in range(bl + bs):
        for q in range(0, len(x), 2 << k):
            if x[q + (1 << k)] is not None:
                x[q] = [x[q], x[q + (1 << k)]]
    return x[0]


def test_fused_leaf_layout_gives_the_two_level_tree():
    for key, tree in GOLD["trees"].items():
        if not key.startswith("_"):
            m, l = (int(v) for v in key.split("x"))
            assert kernel_tree_two_level(m, l) == tree, key
    for m, l in SHAPES + SINGLE + [(1, 2), (1, 5), (1, 8), (1, 32)]:
        if ((m - 1).bit_length() + (l - 1).bit_length()) <= 5 and m <= 8 and l <= 8:     # hand-derived trees: 2 .. 8
            want = TREES1[str(m)] if l == 1 else two_level_tree(m, l) if m > 1 else TREES1[str(l)]
            assert kernel_tree_two_level(m, l) == want, (m, l)


def test_fused_two_level_plan_shape_and_limits():
    base = 0x7f0000000000
    for m, l in SHAPES + SINGLE:
        n = m * l
        uin = [base + r * (1 << 32) for r in range(n)]
        uout = [base + (64 + r) * (1 << 32) for r in range(n)]
        fits = (m - 1).bit_length() + (l - 1).bit_length() <= 5
        for all_reduce, count in ((1, 100003), (0, 4096)):
            if not fits:
                with pytest.raises(h.HcommError) as e:
                    h.OrderPreservedFusedPlan(all_reduce, uin, uout, count, oracle.F32, oracle.SUM, n_servers=m)
                assert e.value.code == h.HcclResult.E_NOT_SUPPORT
                continue
            p = h.OrderPreservedFusedPlan(all_reduce, uin, uout, count, oracle.F32, oracle.SUM, n_servers=m)
            try:
                launches = p.launches()
                assert [x.kind for x in launches] == [h.Kernel.TREE]
                assert launches[0].nseg == (1 if all_reduce else n)
                assert p.info.movedBytes == launches[0].bytes * (2 * n if all_reduce else n + 1)
                ops = (oracle.trace_order_preserved_ar2(oracle.ALG_ALLREDUCE_RING, m, l, count, 1 << 40, oracle.F32) if all_reduce
                       else oracle.trace_order_preserved_rs2(m, l, count, 1 << 40, oracle.F32))
                assert p.info.algorithmicBytes == sum(o[8] * (3 if o[1] else 2) for o in ops)
            finally:
                p.destroy()
    assert not all((m - 1).bit_length() + (l - 1).bit_length() <= 5 for m, l in SHAPES + [(5, 6)])
