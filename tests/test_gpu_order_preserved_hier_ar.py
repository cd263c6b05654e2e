"""GPU parity of the two-level order-preserving allreduce plans (plant + fold in device order inside the servers, plant
+ fold in server order between them, mesh all-gather inside, ring / NB / NHR all-gather between the servers) against
the CPU oracle's transcription of the executor and its templates: user outputs, untouched user inputs and what is left
in both CCL buffers, bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

ALG = {"ring": oracle.ALG_ALLREDUCE_RING, "nhr": oracle.ALG_ALLREDUCE_NHR, "nb": oracle.ALG_ALLREDUCE_NB}

# all-gather between the servers, servers, devices per server, elements, dtype, op, CCL buffer bytes
CASES = [
    ("ring", 2, 8, 1 << 21, "bf16", "sum", 8 << 20),       # one pass, sixteen full blocks
    ("nhr", 4, 4, 300007, "fp32", "sum", 1 << 18),          # 5 chunks, ragged last one
    ("nb", 3, 5, 100003, "fp16", "sum", 1 << 21),           # one pass, short last block
    ("ring", 5, 3, 70001, "int8", "max", 1 << 16),
    ("nhr", 2, 2, 100, "fp32", "prod", 1 << 20),            # blocks of 128, 128, 128 and 16 bytes
    ("nb", 2, 3, 100003, "fp32", "min", 1 << 18),
    ("ring", 8, 4, 50000, "int32", "sum", 1 << 20),
    ("nhr", 7, 3, 4099, "int16", "sum", 1 << 18),
    ("nb", 16, 2, 77777, "bf16", "sum", 1 << 20),
    ("ring", 2, 16, 5, "fp32", "sum", 1 << 17),             # one short block, 31 empty ones
    ("nhr", 3, 2, 0, "fp32", "sum", 4096),
    ("ring", 8, 1, 300007, "fp32", "sum", 1 << 18),        # one device per module: level 0 is a copy into CCL in
    ("nhr", 5, 1, 100003, "bf16", "sum", 1 << 21),
    ("nb", 3, 1, 100, "fp32", "max", 1 << 20),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, alg, m, l, count, dtype, op, ccl, seed=0):
    dt, o, n = DT[dtype], OPS[op], m * l
    host_in = [gen(dt, count, 14000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 998, "wide")
    junk = [np.random.default_rng(17 + i).integers(0, 256, ccl, dtype=np.uint8) for i in range(2)]
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [junk[0].copy() for _ in range(n)]
    w_cout = [junk[1].copy() for _ in range(n)]
    oracle.run_order_preserved_ar2(ALG[alg], m, l, w_in, w_out, w_cin, w_cout, count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cin = [to_dev(junk[0]) for _ in range(n)]
    d_cout = [to_dev(junk[1]) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.OrderPreservedHierAllReducePlan(ALG[alg], m, l, ptrs(d_in), ptrs(d_out), ptrs(d_cin), ptrs(d_cout), ccl, count,
                                             dt, o)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cin[r], junk[0]), w_cin[r]), "CCL in[%d]" % r
            assert np.array_equal(from_dev(d_cout[r], junk[1]), w_cout[r]), "CCL out[%d]" % r
            assert np.array_equal(w_out[r].view(np.uint8), w_out[0].view(np.uint8))      # the same bits on every rank
        ops = oracle.trace_order_preserved_ar2(ALG[alg], m, l, count, ccl, dt)
        assert plan.info.algorithmicBytes == sum(x[8] * (3 if x[1] else 2) for x in ops)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("alg,m,l,count,dtype,op,ccl", CASES)
def test_two_level_order_preserving_allreduce_matches_oracle(gpu_thread, alg, m, l, count, dtype, op, ccl):
    say("order preserved two-level allreduce", alg, m, l, count, dtype, op, ccl)
    run_case(gpu_thread, alg, m, l, count, dtype, op, ccl)


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(6464)
    for i in range(30):
        m = int(rng.integers(2, 9))
        l = int(rng.integers(2, 32 // m + 1))
        alg = ["ring", "nhr", "nb"][rng.integers(3)]
        count = int(rng.integers(1, 400000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        ccl = int(rng.integers(256, 2048)) * 512          # at least 128 KiB: the rounded-up slots always fit
        say("random order preserved two-level allreduce", i, alg, m, l, count, dtype, op, ccl)
        run_case(gpu_thread, alg, m, l, count, dtype, op, ccl, seed=i)


# ---- the single-launch lowering over servers x devices: the same user outputs from one kernel ------------------------

def run_fused(thread, all_reduce, m, l, count, dtype, op, seed=0, kind=None):
    dt, o, n = DT[dtype], OPS[op], m * l
    in_count = count if all_reduce else n * count
    host_in = [gen(dt, in_count, 16000 + seed * 100 + r, kind or ("prod" if op == "prod" else "default")) for r in range(n)]
    sentinel = gen(dt, count, 994, "wide")
    unit = h.DTYPE_SIZE[dt]
    ccl = max(1 << 17, -(-count * unit * n // 128) * 128)
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_ccl = [[np.zeros(ccl, np.uint8) for _ in range(n)] for _ in range(2)]
    if all_reduce:
        oracle.run_order_preserved_ar2(oracle.ALG_ALLREDUCE_NHR, m, l, w_in, w_out, w_ccl[0], w_ccl[1], count, ccl, dt, o)
    else:
        oracle.run_order_preserved_rs2(m, l, w_in, w_out, w_ccl[0], w_ccl[1], count, ccl, dt, o)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    plan = h.OrderPreservedFusedPlan(all_reduce, [t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out], count, dt, o,
                                     n_servers=m)
    try:
        assert plan.info.launches == 1
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
    finally:
        plan.destroy()


FUSED_CASES = [
    (1, 2, 8, 1 << 20, "bf16", "sum"),
    (1, 4, 4, 300007, "fp32", "sum"),
    (1, 3, 5, 100003, "fp16", "sum"),          # 4 x 8 leaf positions, 17 holes
    (1, 5, 3, 70001, "int8", "max"),
    (1, 2, 2, 100, "fp32", "prod"),
    (1, 8, 4, 50000, "int32", "sum"),
    (1, 7, 3, 4099, "int16", "sum"),
    (1, 16, 2, 77777, "bf16", "sum"),
    (1, 2, 16, 33333, "fp32", "min"),
    (0, 2, 8, 1 << 16, "bf16", "sum"),
    (0, 4, 4, 100000, "fp32", "sum"),
    (0, 3, 5, 30000, "fp16", "sum"),
    (0, 7, 3, 4104, "int16", "sum"),
    (0, 2, 2, 16, "fp32", "prod"),
    (1, 8, 1, 100003, "fp32", "sum"),          # one device per module
    (0, 5, 1, 4096, "bf16", "sum"),
]


@pytest.mark.parametrize("all_reduce,m,l,count,dtype,op", FUSED_CASES)
def test_single_launch_lowering_matches_the_two_level_executors(gpu_thread, all_reduce, m, l, count, dtype, op):
    say("order preserved two-level fused", all_reduce, m, l, count, dtype, op)
    run_fused(gpu_thread, all_reduce, m, l, count, dtype, op)


def test_single_launch_lowering_randomized(gpu_thread):
    rng = np.random.default_rng(6666)
    done = 0
    while done < 30:
        all_reduce = int(rng.integers(2))
        m = int(rng.integers(2, 9))
        l = int(rng.integers(2, 32 // m + 1))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        unit = h.DTYPE_SIZE[DT[dtype]]
        count = int(rng.integers(1, 100000))
        if (m - 1).bit_length() + (l - 1).bit_length() > 5:
            continue                                          # more than 32 leaf positions: no single-launch plan
        if not all_reduce:
            count = max(16 // unit, count // 8 // (16 // unit) * (16 // unit))   # blocks of whole 16 bytes
        op = ["sum", "max", "min"][rng.integers(3)]
        say("random order preserved two-level fused", done, all_reduce, m, l, count, dtype, op)
        run_fused(gpu_thread, all_reduce, m, l, count, dtype, op, seed=done)
        done += 1


@pytest.mark.parametrize("dtype,op", [("fp16", "sum"), ("fp16", "max"), ("fp16", "min"), ("bf16", "sum"), ("bf16", "max"),
                                      ("bf16", "min"), ("fp32", "min")])
def test_single_launch_lowering_on_every_bit_pattern(gpu_thread, dtype, op):
    """NaNs, infinities, signed zeros and denormals through both levels of the tree: MAX / MIN keep the operand in the
    dst role on a tie or a NaN, which pins the side of every fold."""
    for all_reduce, m, l, count in ((1, 2, 8, 70000), (1, 3, 5, 30001), (0, 4, 4, 4096), (0, 2, 3, 8192)):
        say("order preserved two-level fused, wide values", all_reduce, m, l, count, dtype, op)
        run_fused(gpu_thread, all_reduce, m, l, count, dtype, op, seed=78, kind="wide")
