"""GPU parity of the two-level order-preserving reduce-scatter plans (plant + fold in device order inside the servers,
plant + fold in server order between them, own block to the user output) against the CPU oracle's transcription of the
executor and its templates: user outputs, untouched user inputs and what is left in the CCL output buffers, bit for
bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

# servers, devices per server, elements per block, dtype, op, CCL buffer bytes
CASES = [
    (2, 8, 1 << 17, "bf16", "sum", 8 << 20),       # one pass, aligned blocks
    (4, 4, 100007, "fp32", "sum", 1 << 20),        # 7 chunks, ragged last one
    (3, 5, 30001, "fp16", "sum", 1 << 21),         # one pass, blocks at odd byte offsets
    (5, 3, 7001, "int8", "max", 1 << 16),
    (2, 2, 10, "fp32", "prod", 1 << 20),
    (2, 3, 50003, "fp32", "min", 1 << 18),
    (8, 4, 5000, "int32", "sum", 1 << 20),
    (7, 3, 4099, "int16", "sum", 1 << 18),
    (16, 2, 7777, "bf16", "sum", 1 << 20),
    (3, 2, 0, "fp32", "sum", 4096),
    (8, 1, 100007, "fp32", "sum", 1 << 20),        # one device per module: the blocks are staged in CCL in
    (5, 1, 30001, "bf16", "sum", 1 << 21),
    (3, 1, 10, "fp32", "max", 1 << 20),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, m, l, count, dtype, op, ccl, seed=0):
    dt, o, n = DT[dtype], OPS[op], m * l
    host_in = [gen(dt, n * count, 15000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 999, "wide")
    junk = np.random.default_rng(19).integers(0, 256, ccl, dtype=np.uint8)
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [junk[::-1].copy() for _ in range(n)]
    w_cout = [junk.copy() for _ in range(n)]
    oracle.run_order_preserved_rs2(m, l, w_in, w_out, w_cin, w_cout, count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cin = [to_dev(junk[::-1].copy()) for _ in range(n)]
    d_cout = [to_dev(junk) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.OrderPreservedHierReduceScatterPlan(m, l, ptrs(d_in), ptrs(d_out), ptrs(d_cout), ccl, count, dt, o,
                                                 ccl_in=ptrs(d_cin) if l == 1 else None)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cout[r], junk), w_cout[r]), "CCL out[%d]" % r
            assert np.array_equal(from_dev(d_cin[r], junk), w_cin[r]), "CCL in[%d]" % r
        ops = oracle.trace_order_preserved_rs2(m, l, count, ccl, dt)
        assert plan.info.algorithmicBytes == sum(x[8] * (3 if x[1] else 2) for x in ops)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("m,l,count,dtype,op,ccl", CASES)
def test_two_level_order_preserving_reduce_scatter_matches_oracle(gpu_thread, m, l, count, dtype, op, ccl):
    say("order preserved two-level reduce-scatter", m, l, count, dtype, op, ccl)
    run_case(gpu_thread, m, l, count, dtype, op, ccl)


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(6565)
    for i in range(30):
        m = int(rng.integers(2, 9))
        l = int(rng.integers(2, 32 // m + 1))
        count = int(rng.integers(1, 30000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        ccl = int(rng.integers(1, 64)) * 128 * m * l * 4
        say("random order preserved two-level reduce-scatter", i, m, l, count, dtype, op, ccl)
        run_case(gpu_thread, m, l, count, dtype, op, ccl, seed=i)
