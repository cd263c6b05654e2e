"""The op-base loop around the templates (user buffers -> CCL buffers -> template -> user buffers): the oracle's
transcription of the executors' RunLoop / RunLoopInner against hand-derived chunk tables, against exact integer
arithmetic, against the symbolic checker and against the product's independent generator."""
import json
import os

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import Expect

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedules_hand_derived.json")))["opbase_loop"]
ALG = {"ring_ar": oracle.ALG_ALLREDUCE_RING, "mesh_rs": oracle.ALG_RS_MESH}
ALLREDUCE = [oracle.ALG_ALLREDUCE_RING, oracle.ALG_ALLREDUCE_RHD, oracle.ALG_ALLREDUCE_MESH_ONESHOT,
             oracle.ALG_ALLREDUCE_MESH_ASCENDING, oracle.ALG_ALLREDUCE_LOCAL_REDUCE, oracle.ALG_ALLREDUCE_CHUNK_MESH,
             oracle.ALG_ALLREDUCE_NHR, oracle.ALG_ALLREDUCE_NB, oracle.ALG_ALLREDUCE_DOUBLING,
             oracle.ALG_ALLREDUCE_NHR_ONESHOT]
POW2_ONLY = (oracle.ALG_ALLREDUCE_LOCAL_REDUCE, oracle.ALG_ALLREDUCE_DOUBLING)
SCATTER = [oracle.ALG_RS_MESH, oracle.ALG_RS_RING_STANDALONE, oracle.ALG_RS_NHR, oracle.ALG_RS_NB,
           oracle.ALG_RS_LOCAL_REDUCE]
UIN, UOUT = 3, 4


def test_chunk_tables_hand_derived():
    for case in GOLD["cases"]:
        alg, n, count, unit, ccl = ALG[case["alg"]], case["n"], case["count"], case["unit"], case["ccl_bytes"]
        dt = {4: oracle.F32, 1: oracle.I8}[unit]
        assert oracle.opbase_max_count(alg, n, ccl, dt) == case["max_count"]
        assert h.opbase_max_count(alg, n, ccl, dt) == case["max_count"]
        ops = oracle.trace_opbase(alg, n, count, ccl, dt)
        outs = sorted((o[4], o[8]) for o in ops if o[3] == UOUT and o[2] == 0)        # copies to rank 0's user output
        assert [list(x) for x in outs] == case["chunks"]
        ins = [o for o in ops if o[6] == UIN and o[2] == 0]
        steps = sorted(set(o[0] for o in ins))
        got = [[[o[4], o[7], o[8]] for o in ins if o[0] == s] for s in steps]
        assert got == case["copies_in_rank0"]
        for o in ops:                                                                  # the loop only ever copies
            if o[3] in (UIN, UOUT) or o[6] in (UIN, UOUT):
                assert o[1] == 0 and o[2] == o[5]
    d = GOLD["max_count_defaults"]
    ccl = 200 << 20
    assert oracle.opbase_max_count(oracle.ALG_ALLREDUCE_RING, 8, ccl, oracle.BF16) == d["ring_ar_bf16"]
    assert oracle.opbase_max_count(oracle.ALG_RS_RING_STANDALONE, 8, ccl, oracle.F32) == d["rs_n8_fp32"]
    assert oracle.opbase_max_count(oracle.ALG_RS_MESH, 7, ccl, oracle.I8) == d["rs_n7_int8"]


CONFIGS = [(1000, oracle.F32, 2048), (1000, oracle.F32, 1 << 20), (100003, oracle.I8, 60000), (0, oracle.F32, 4096),
           (77777, oracle.F32, 200000)]


@pytest.mark.parametrize("alg", ALLREDUCE + SCATTER)
def test_product_generator_equals_oracle_trace_and_passes_the_checker(alg):
    expect = Expect.REDUCE_SCATTER_USER if alg in SCATTER else Expect.ALLREDUCE_USER
    for n in (1, 2, 3, 4, 5, 8, 16):
        if alg in POW2_ONLY and n & (n - 1):
            continue
        for count, dt, ccl in CONFIGS + [(5, oracle.F16, 128 * n)]:
            if oracle.opbase_max_count(alg, n, ccl, dt) == 0:              # the executors refuse such a buffer
                with pytest.raises(ValueError):
                    oracle.trace_opbase(alg, n, count, ccl, dt)
                with pytest.raises(h.HcommError):
                    h.opbase_emit(alg, n, count, ccl, dt)
                continue
            a = oracle.trace_opbase(alg, n, count, ccl, dt)
            assert a == h.opbase_emit(alg, n, count, ccl, dt), (alg, n, count, ccl)
            assert h.opbase_check(alg, n, count, ccl, dt)[:2] == (0, 0), (alg, n, count, ccl)
            assert h.oplist_check(a, n, expect, count, h.DTYPE_SIZE[dt])[:2] == (0, 0), (alg, n, count, ccl)


def test_rejects_what_the_executors_reject():
    for f in (oracle.trace_opbase, h.opbase_emit):
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_ALLREDUCE_RING, 4, 100, 3, oracle.F32)          # CCL buffer smaller than one element
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_RS_MESH, 4, 100, 500, oracle.F32)               # no 128-byte slice per rank fits
        with pytest.raises((ValueError, h.HcommError)):
            f(oracle.ALG_RS_RING_STAGE, 4, 100, 4096, oracle.F32)        # the in-place stage has no executor loop


def scratch_for(alg, n, count, ccl, dt):
    chunk = min(count, oracle.opbase_max_count(alg, n, ccl, dt))
    sb = h.scratch_bytes(alg, n, chunk, dt) if chunk else 0
    return [np.zeros(sb, np.uint8) for _ in range(n)] if sb else None


@pytest.mark.parametrize("alg", ALLREDUCE + SCATTER)
@pytest.mark.parametrize("n", [1, 2, 3, 4, 7, 8])
def test_exact_integer_results_through_the_loop(alg, n):
    """Chunked or not, every element of the user output is the exact int32 sum (MAX) over the ranks."""
    if alg in POW2_ONLY and n & (n - 1):
        pytest.skip("power-of-two rank counts only")
    count = 5003
    scatter = alg in SCATTER
    rng = np.random.default_rng(alg * 100 + n)
    for ccl in (4096 * n, 1 << 22):                                       # several chunks / one pass
        per_in = n * count if scatter else count
        ins = [rng.integers(-1 << 20, 1 << 20, per_in).astype(np.int32) for _ in range(n)]
        for op, fold in ((oracle.SUM, lambda xs: np.sum(xs, axis=0, dtype=np.int64).astype(np.int32)),
                         (oracle.MAX, lambda xs: np.max(xs, axis=0))):
            outs = [np.full(count, -7, np.int32) for _ in range(n)]
            cin = [np.full(ccl // 4, -1, np.int32) for _ in range(n)]
            cout = [np.full(ccl // 4, -2, np.int32) for _ in range(n)]
            before = [x.copy() for x in ins]
            oracle.run_opbase(alg, ins, outs, cin, cout, count, ccl, oracle.I32, op,
                              scratch=scratch_for(alg, n, count, ccl, oracle.I32))
            want = fold(np.stack(before))
            for r in range(n):
                assert np.array_equal(ins[r], before[r]), "the loop never writes the user input"
                w = want[r * count:(r + 1) * count] if scatter else want
                assert np.array_equal(outs[r], w), (alg, n, ccl, op, r)


def test_algorithmic_bytes_add_the_two_copies():
    """One pass: the template's bytes + 2 * S in + 2 * S out per rank (allreduce)."""
    n, count = 8, 1 << 20
    base = oracle.algorithmic_bytes(oracle.ALG_ALLREDUCE_RING, n, count, oracle.BF16)
    got = oracle.algorithmic_bytes_opbase(oracle.ALG_ALLREDUCE_RING, n, count, 200 << 20, oracle.BF16)
    assert got == base + 4 * n * count * 2
