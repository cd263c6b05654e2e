"""GPU parity of the double-ring allreduce plans (op-base mode with DMA reduce: user buffers read and written directly)
against the CPU oracle's transcription of the executor and its two templates: user outputs, untouched user inputs and
what is left in both CCL buffers, bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

LEVEL1 = {"ring": oracle.ALG_ALLREDUCE_RING, "nhr": oracle.ALG_ALLREDUCE_NHR, "nb": oracle.ALG_ALLREDUCE_NB}

# level-1 algorithm, servers, ranks per server, elements, dtype, op, CCL buffer bytes
CASES = [
    ("ring", 1, 8, 1 << 20, "bf16", "sum", 8 << 20),       # one server, one pass
    ("ring", 1, 8, 1000003, "fp32", "sum", 1 << 20),       # 4 chunks, ragged last one
    ("nhr", 2, 8, 1 << 21, "bf16", "sum", 8 << 20),        # sliced NHR between two servers
    ("nhr", 4, 4, 100003, "fp16", "sum", 1 << 20),         # one-shot NHR between four servers
    ("nb", 3, 5, 300007, "int32", "max", 1 << 19),
    ("ring", 2, 16, 70001, "int8", "sum", 1 << 16),
    ("ring", 1, 3, 192, "fp32", "prod", 4096),
    ("ring", 1, 2, 100003, "fp32", "min", 1 << 18),
    ("ring", 1, 1, 1000, "fp32", "sum", 2048),             # one rank: user in -> CCL in -> CCL out -> user out
    ("nb", 8, 1, 100003, "int16", "sum", 1 << 17),         # one rank per server: the level-1 template between copies
    ("ring", 1, 16, 9, "int32", "sum", 4096),              # most shares empty
    ("ring", 1, 4, 0, "fp32", "sum", 4096),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, alg1, ns, nl, count, dtype, op, ccl, seed=0):
    dt, o, n = DT[dtype], OPS[op], ns * nl
    host_in = [gen(dt, count, 9000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 996, "wide")
    junk = np.random.default_rng(13).integers(0, 256, ccl, dtype=np.uint8)
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [junk.copy() for _ in range(n)]
    w_cout = [junk[::-1].copy() for _ in range(n)]
    oracle.run_dbring(LEVEL1[alg1], ns, nl, w_in, w_out, w_cin, w_cout, count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cin = [to_dev(junk) for _ in range(n)]
    d_cout = [to_dev(junk[::-1].copy()) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.DoubleRingPlan(LEVEL1[alg1], ns, nl, ptrs(d_in), ptrs(d_out), ptrs(d_cin), ptrs(d_cout), ccl, count, dt, o)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cin[r], junk), w_cin[r]), "CCL in[%d]" % r
            assert np.array_equal(from_dev(d_cout[r], junk), w_cout[r]), "CCL out[%d]" % r
        ops = oracle.trace_dbring(LEVEL1[alg1], ns, nl, count, ccl, dt)
        assert plan.info.algorithmicBytes == sum(x[8] * (3 if x[1] else 2) for x in ops)
        assert plan.info.movedBytes == plan.info.algorithmicBytes
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("alg1,ns,nl,count,dtype,op,ccl", CASES)
def test_double_ring_allreduce_matches_oracle(gpu_thread, alg1, ns, nl, count, dtype, op, ccl):
    say("double ring", alg1, ns, nl, count, dtype, op, ccl)
    run_case(gpu_thread, alg1, ns, nl, count, dtype, op, ccl)


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(5151)
    names = sorted(LEVEL1)
    for i in range(40):
        alg1 = names[rng.integers(len(names))]
        ns, nl = int(rng.integers(1, 5)), int(rng.integers(1, 17))
        if ns * nl > 32:
            ns = 32 // nl
        count = int(rng.integers(1, 300000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        ccl = int(rng.integers(1, 64)) * 4096
        say("random double ring", i, alg1, ns, nl, count, dtype, op, ccl)
        run_case(gpu_thread, alg1, ns, nl, count, dtype, op, ccl, seed=i)
