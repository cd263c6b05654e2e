"""GPU parity of the double-ring reduce-scatter plans (one server, op-base mode with DMA reduce) against the CPU oracle's
transcription of the executor and its template: user outputs, untouched user inputs and what is left in the CCL input
buffers, bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

# ranks, elements per block, dtype, op, CCL buffer bytes
CASES = [
    (8, 1 << 18, "bf16", "sum", 8 << 20),      # one pass
    (8, 300007, "fp32", "sum", 1 << 20),       # 10 chunks, ragged last one
    (7, 100003, "fp16", "sum", 1 << 21),       # blocks at odd byte offsets of the user input
    (5, 70001, "int8", "max", 1 << 16),
    (3, 64, "fp32", "prod", 1 << 20),
    (16, 4099, "int16", "sum", 1 << 18),
    (32, 5000, "int32", "min", 1 << 20),
    (4, 9, "int32", "sum", 4096),              # second shares empty
    (6, 0, "fp32", "sum", 4096),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, n, count, dtype, op, ccl, seed=0):
    dt, o = DT[dtype], OPS[op]
    host_in = [gen(dt, n * count, 15000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 993, "wide")
    junk = np.random.default_rng(16).integers(0, 256, ccl, dtype=np.uint8)
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [junk.copy() for _ in range(n)]
    oracle.run_dbring_rs(w_in, w_out, w_cin, count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cin = [to_dev(junk) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.DoubleRingReduceScatterPlan(ptrs(d_in), ptrs(d_out), ptrs(d_cin), ccl, count, dt, o)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cin[r], junk), w_cin[r]), "CCL in[%d]" % r
        ops = oracle.trace_dbring_rs(n, count, ccl, dt)
        assert plan.info.algorithmicBytes == sum(x[8] * (3 if x[1] else 2) for x in ops)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("n,count,dtype,op,ccl", CASES)
def test_double_ring_reduce_scatter_matches_oracle(gpu_thread, n, count, dtype, op, ccl):
    say("double ring rs", n, count, dtype, op, ccl)
    run_case(gpu_thread, n, count, dtype, op, ccl)


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(8181)
    for i in range(30):
        n = int(rng.integers(3, 17))
        count = int(rng.integers(1, 100000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        ccl = int(rng.integers(1, 64)) * 128 * n * 4
        say("random double ring rs", i, n, count, dtype, op, ccl)
        run_case(gpu_thread, n, count, dtype, op, ccl, seed=i)
