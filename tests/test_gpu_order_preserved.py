"""GPU parity of the order-preserving reduce-scatter plans (plant into the peers' CCL output buffers, fold in rank
order, own slot to the user output) against the CPU oracle's transcription of the executor and its template: user
outputs, untouched user inputs and what is left in the CCL output buffers, bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

# ranks, elements per block, dtype, op, CCL buffer bytes
CASES = [
    (8, 1 << 18, "bf16", "sum", 8 << 20),      # one pass, aligned slots
    (8, 300007, "fp32", "sum", 1 << 20),       # 10 chunks, ragged last one
    (7, 100003, "fp16", "sum", 1 << 21),       # one pass, slots at odd byte offsets
    (5, 70001, "int8", "max", 1 << 16),
    (3, 10, "fp32", "prod", 1 << 20),
    (2, 100003, "fp32", "min", 1 << 18),
    (16, 4099, "int16", "sum", 1 << 18),
    (32, 5000, "int32", "sum", 1 << 20),
    (6, 0, "fp32", "sum", 4096),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, n, count, dtype, op, ccl, seed=0):
    dt, o = DT[dtype], OPS[op]
    host_in = [gen(dt, n * count, 11000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 995, "wide")
    junk = np.random.default_rng(14).integers(0, 256, ccl, dtype=np.uint8)
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [np.zeros(16, np.uint8) for _ in range(n)]
    w_cout = [junk.copy() for _ in range(n)]
    oracle.run_order_preserved(w_in, w_out, w_cin, w_cout, count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cout = [to_dev(junk) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.OrderPreservedPlan(ptrs(d_in), ptrs(d_out), ptrs(d_cout), ccl, count, dt, o)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cout[r], junk), w_cout[r]), "CCL out[%d]" % r
        ops = oracle.trace_order_preserved(n, count, ccl, dt)
        assert plan.info.algorithmicBytes == sum(x[8] * (3 if x[1] else 2) for x in ops)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("n,count,dtype,op,ccl", CASES)
def test_order_preserving_reduce_scatter_matches_oracle(gpu_thread, n, count, dtype, op, ccl):
    say("order preserved", n, count, dtype, op, ccl)
    run_case(gpu_thread, n, count, dtype, op, ccl)


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(6161)
    for i in range(30):
        n = int(rng.integers(2, 17))
        count = int(rng.integers(1, 100000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        ccl = int(rng.integers(1, 64)) * 128 * n * 4
        say("random order preserved", i, n, count, dtype, op, ccl)
        run_case(gpu_thread, n, count, dtype, op, ccl, seed=i)


# ---- the executor's branch for small messages (ReduceScatterHDStage, 4 or 8 ranks, at most 32 KiB per rank) -----------

def run_small(thread, n, count, dtype, op, ccl, seed=0):
    dt, o = DT[dtype], OPS[op]
    host_in = [gen(dt, n * count, 17000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 993, "wide")
    junk = np.random.default_rng(21).integers(0, 256, ccl, dtype=np.uint8)
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [np.zeros(16, np.uint8) for _ in range(n)]
    w_cout = [junk.copy() for _ in range(n)]
    oracle.run_order_preserved_small(w_in, w_out, w_cin, w_cout, count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cout = [to_dev(junk) for _ in range(n)]
    plan = h.OrderPreservedSmallPlan([t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out],
                                     [t.data_ptr() for t in d_cout], ccl, count, dt, o)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cout[r], junk), w_cout[r]), "CCL out[%d]" % r
        steps = 2 + n.bit_length() - 1
        # one launch per step; two where blocks off 16-byte boundaries need the element-wise kernel beside the vector one
        assert plan.info.launches == steps if count * h.DTYPE_SIZE[dt] % 16 == 0 else steps <= plan.info.launches <= 2 * steps
    finally:
        plan.destroy()


@pytest.mark.parametrize("n,count,dtype,op", [
    (8, 16384, "bf16", "sum"),      # 32 KiB per rank
    (8, 8192, "fp32", "sum"),
    (4, 16384, "fp16", "sum"),
    (8, 32768, "int8", "max"),
    (4, 4, "fp32", "prod"),
    (8, 1001, "fp32", "min"),       # blocks at offsets that are not 16-byte multiples
    (4, 333, "int16", "sum"),
    (8, 1, "int32", "sum"),
])
def test_small_message_branch_matches_oracle(gpu_thread, n, count, dtype, op):
    say("order preserved small", n, count, dtype, op)
    run_small(gpu_thread, n, count, dtype, op, 1 << 20)


def test_small_message_branch_randomized(gpu_thread):
    rng = np.random.default_rng(6767)
    for i in range(30):
        n = [4, 8][rng.integers(2)]
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        count = int(rng.integers(1, 32768 // h.DTYPE_SIZE[DT[dtype]] + 1))
        op = ["sum", "max", "min"][rng.integers(3)]
        say("random order preserved small", i, n, count, dtype, op)
        run_small(gpu_thread, n, count, dtype, op, n * 32768, seed=i)
