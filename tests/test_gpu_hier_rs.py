"""GPU parity of the two-level reduce-scatter plans (ring and mesh executors in op-base mode) against the CPU oracle's
transcription: user outputs, untouched user inputs and what is left in both CCL buffers, bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

LEVEL1 = {"ring": (oracle.ALG_RS_RING_STAGE, h.Alg.REDUCE_SCATTER_RING), "nhr": (oracle.ALG_RS_NHR, h.Alg.REDUCE_SCATTER_NHR),
          "nb": (oracle.ALG_RS_NB, h.Alg.REDUCE_SCATTER_NB), "rhd": (oracle.ALG_RS_RHD, h.Alg.REDUCE_SCATTER_RHD)}

# level 0 (mesh?), level-1 algorithm, servers, ranks per server, elements per block, dtype, op, CCL buffer bytes
CASES = [
    (False, "ring", 1, 8, 1 << 17, "bf16", "sum", 8 << 20),     # one server, one pass: a single copy in
    (False, "ring", 2, 8, 100003, "fp32", "sum", 1 << 22),      # 2 chunks
    (False, "nhr", 4, 4, 70001, "fp16", "sum", 1 << 20),
    (False, "nb", 3, 5, 30007, "int32", "max", 1 << 19),
    (False, "ring", 2, 1, 100003, "int16", "sum", 1 << 18),     # one rank per server: level 1 alone
    (True, "ring", 1, 8, 1 << 17, "bf16", "sum", 8 << 20),
    (True, "nhr", 2, 8, 100003, "fp32", "sum", 1 << 22),
    (True, "nb", 5, 3, 70001, "int8", "sum", 1 << 18),
    (True, "ring", 1, 2, 10, "fp32", "prod", 4096),
    (True, "ring", 2, 16, 4099, "fp32", "min", 1 << 20),
    (False, "ring", 4, 8, 9, "int32", "sum", 1 << 16),
    (True, "ring", 2, 4, 0, "fp32", "sum", 4096),
    (False, "rhd", 6, 2, 70001, "fp32", "sum", 1 << 21),       # recursive halving-doubling between 6 servers
    (True, "rhd", 4, 4, 30007, "bf16", "sum", 1 << 20),
    (False, "rhd", 17, 1, 10003, "int32", "max", 1 << 20),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, mesh, alg1, ns, nl, count, dtype, op, ccl, seed=0):
    dt, o, n = DT[dtype], OPS[op], ns * nl
    host_in = [gen(dt, n * count, 13000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 994, "wide")
    junk = np.random.default_rng(15).integers(0, 256, ccl, dtype=np.uint8)
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [junk.copy() for _ in range(n)]
    w_cout = [junk[::-1].copy() for _ in range(n)]
    oracle.run_hier_rs(LEVEL1[alg1][0], ns, nl, w_in, w_out, w_cin, w_cout, count, ccl, dt, o, mesh=mesh)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cin = [to_dev(junk) for _ in range(n)]
    d_cout = [to_dev(junk[::-1].copy()) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.HierReduceScatterPlan(LEVEL1[alg1][1], ns, nl, ptrs(d_in), ptrs(d_out), ptrs(d_cin), ptrs(d_cout), ccl, count,
                                   dt, o, mesh=mesh)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cin[r], junk), w_cin[r]), "CCL in[%d]" % r
            assert np.array_equal(from_dev(d_cout[r], junk), w_cout[r]), "CCL out[%d]" % r
        ops = oracle.trace_hier_rs(LEVEL1[alg1][0], ns, nl, count, ccl, dt, mesh=mesh)
        assert plan.info.algorithmicBytes == sum(x[8] * (3 if x[1] else 2) for x in ops)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("mesh,alg1,ns,nl,count,dtype,op,ccl", CASES)
def test_two_level_reduce_scatter_matches_oracle(gpu_thread, mesh, alg1, ns, nl, count, dtype, op, ccl):
    say("hier rs", mesh, alg1, ns, nl, count, dtype, op, ccl)
    run_case(gpu_thread, mesh, alg1, ns, nl, count, dtype, op, ccl)


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(7171)
    names = sorted(LEVEL1)
    for i in range(30):
        alg1 = names[rng.integers(len(names))]
        ns, nl = int(rng.integers(1, 5)), int(rng.integers(1, 9))
        mesh = bool(rng.integers(2)) and nl >= 2
        count = int(rng.integers(1, 50000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        ccl = int(rng.integers(1, 64)) * 512 * ns * nl
        say("random hier rs", i, mesh, alg1, ns, nl, count, dtype, op, ccl)
        run_case(gpu_thread, mesh, alg1, ns, nl, count, dtype, op, ccl, seed=i)
