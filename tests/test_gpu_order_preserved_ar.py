"""GPU parity of the order-preserving allreduce plans (plant with one slot borrowed from the CCL input buffer, fold in
rank order, mesh all-gather inside the CCL output buffers, chunk to the user output) against the CPU oracle's
transcription of the executor and its templates: user outputs, untouched user inputs and what is left in both CCL
buffers, bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

# ranks, elements, dtype, op, CCL buffer bytes
CASES = [
    (8, 1 << 21, "bf16", "sum", 8 << 20),      # one pass, eight full blocks
    (8, 300007, "fp32", "sum", 1 << 18),       # 5 chunks, ragged last one
    (7, 100003, "fp16", "sum", 1 << 21),       # one pass, short last block
    (5, 70001, "int8", "max", 1 << 16),
    (3, 100, "fp32", "prod", 1 << 20),         # blocks of 256, 144 and 0 bytes
    (2, 100003, "fp32", "min", 1 << 18),
    (16, 4099, "int16", "sum", 1 << 18),
    (32, 50000, "int32", "sum", 1 << 20),
    (8, 5, "fp32", "sum", 1 << 16),            # one short block, seven empty ones
    (6, 0, "fp32", "sum", 4096),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, n, count, dtype, op, ccl, seed=0):
    dt, o = DT[dtype], OPS[op]
    host_in = [gen(dt, count, 12000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 996, "wide")
    junk = [np.random.default_rng(15 + i).integers(0, 256, ccl, dtype=np.uint8) for i in range(2)]
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [junk[0].copy() for _ in range(n)]
    w_cout = [junk[1].copy() for _ in range(n)]
    oracle.run_order_preserved_ar(w_in, w_out, w_cin, w_cout, count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cin = [to_dev(junk[0]) for _ in range(n)]
    d_cout = [to_dev(junk[1]) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.OrderPreservedAllReducePlan(ptrs(d_in), ptrs(d_out), ptrs(d_cin), ptrs(d_cout), ccl, count, dt, o)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cin[r], junk[0]), w_cin[r]), "CCL in[%d]" % r
            assert np.array_equal(from_dev(d_cout[r], junk[1]), w_cout[r]), "CCL out[%d]" % r
            assert np.array_equal(w_out[r].view(np.uint8), w_out[0].view(np.uint8))      # the same bits on every rank
        ops = oracle.trace_order_preserved_ar(n, count, ccl, dt)
        assert plan.info.algorithmicBytes == sum(x[8] * (3 if x[1] else 2) for x in ops)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("n,count,dtype,op,ccl", CASES)
def test_order_preserving_allreduce_matches_oracle(gpu_thread, n, count, dtype, op, ccl):
    say("order preserved allreduce", n, count, dtype, op, ccl)
    run_case(gpu_thread, n, count, dtype, op, ccl)


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(6262)
    for i in range(30):
        n = int(rng.integers(2, 17))
        count = int(rng.integers(1, 400000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        ccl = int(rng.integers(64, 2048)) * 512           # at least 32 KiB: the N - 1 rounded-up slots always fit
        say("random order preserved allreduce", i, n, count, dtype, op, ccl)
        run_case(gpu_thread, n, count, dtype, op, ccl, seed=i)


# ---- the single-launch lowering: the same user outputs from one kernel that only reads the user inputs ---------------

def run_fused(thread, all_reduce, n, count, dtype, op, seed=0, kind=None):
    dt, o = DT[dtype], OPS[op]
    in_count = count if all_reduce else n * count
    host_in = [gen(dt, in_count, 13000 + seed * 100 + r, kind or ("prod" if op == "prod" else "default")) for r in range(n)]
    sentinel = gen(dt, count, 997, "wide")
    unit = h.DTYPE_SIZE[dt]
    ccl = max(4096, -(-count * unit * n // 128) * 128)            # one chunk or several: the result does not depend on it
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_ccl = [[np.zeros(ccl, np.uint8) for _ in range(n)] for _ in range(2)]
    if all_reduce:
        oracle.run_order_preserved_ar(w_in, w_out, w_ccl[0], w_ccl[1], count, ccl, dt, o)
    else:
        oracle.run_order_preserved(w_in, w_out, w_ccl[0], w_ccl[1], count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.OrderPreservedFusedPlan(all_reduce, ptrs(d_in), ptrs(d_out), count, dt, o)
    try:
        assert plan.info.launches == (1 if count else 0)
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
    finally:
        plan.destroy()


FUSED_CASES = [
    (1, 8, 1 << 21, "bf16", "sum"),
    (1, 8, 300007, "fp32", "sum"),
    (1, 7, 100003, "fp16", "sum"),
    (1, 5, 70001, "int8", "max"),
    (1, 3, 100, "fp32", "prod"),
    (1, 2, 100003, "fp32", "min"),
    (1, 16, 4099, "int16", "sum"),
    (1, 32, 50000, "int32", "sum"),
    (1, 13, 77777, "bf16", "sum"),
    (1, 6, 0, "fp32", "sum"),
    (0, 8, 1 << 18, "bf16", "sum"),
    (0, 7, 100000, "fp16", "sum"),
    (0, 5, 70000, "fp32", "prod"),
    (0, 3, 16, "int8", "max"),
    (0, 32, 5000, "int32", "sum"),
    (0, 12, 4104, "int16", "min"),
]


@pytest.mark.parametrize("all_reduce,n,count,dtype,op", FUSED_CASES)
def test_single_launch_lowering_matches_the_executors_outputs(gpu_thread, all_reduce, n, count, dtype, op):
    say("order preserved fused", all_reduce, n, count, dtype, op)
    run_fused(gpu_thread, all_reduce, n, count, dtype, op)


def test_single_launch_lowering_randomized(gpu_thread):
    rng = np.random.default_rng(6363)
    for i in range(40):
        all_reduce = int(rng.integers(2))
        n = int(rng.integers(2, 33))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        unit = h.DTYPE_SIZE[DT[dtype]]
        count = int(rng.integers(1, 200000))
        if not all_reduce:
            count = max(16 // unit, count // 4 // (16 // unit) * (16 // unit))   # blocks of whole 16 bytes
        op = ["sum", "max", "min"][rng.integers(3)]
        say("random order preserved fused", i, all_reduce, n, count, dtype, op)
        run_fused(gpu_thread, all_reduce, n, count, dtype, op, seed=i)


@pytest.mark.parametrize("dtype,op", [("fp16", "sum"), ("fp16", "max"), ("fp16", "min"), ("fp16", "prod"), ("bf16", "sum"),
                                      ("bf16", "max"), ("bf16", "min"), ("fp32", "max"), ("fp32", "sum")])
def test_single_launch_lowering_on_every_bit_pattern(gpu_thread, dtype, op):
    """NaNs, infinities, signed zeros and denormals: MAX / MIN keep the operand in the dst role on a tie or a NaN, so
    this also pins which side of every fold of the tree is which."""
    for all_reduce, n, count in ((1, 8, 70000), (1, 5, 70001), (0, 8, 8192), (0, 3, 4096)):
        say("order preserved fused, wide values", all_reduce, n, count, dtype, op)
        run_fused(gpu_thread, all_reduce, n, count, dtype, op, seed=77, kind="wide")
