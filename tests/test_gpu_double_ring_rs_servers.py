"""GPU parity of the double-ring reduce-scatter plans over several servers and super pods (op-base mode with DMA reduce;
ring, NHR or NB between the servers of a pod and between the pods) against the CPU oracle's transcription of the executor and its templates: user outputs, untouched
user inputs and what is left in the CCL input buffers, bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

ALG = {"ring": oracle.ALG_RS_RING_STAGE, "nhr": oracle.ALG_RS_NHR, "nb": oracle.ALG_RS_NB}

# level-1 algorithm, servers, devices per server, elements per block, dtype, op, CCL buffer bytes
CASES = [
    ("ring", 2, 8, 1 << 17, "bf16", "sum", 8 << 20),    # one pass
    ("nhr", 4, 8, 50021, "fp32", "sum", 1 << 21),       # 4 chunks, ragged last one
    ("nb", 3, 5, 100003, "fp16", "sum", 1 << 21),       # blocks at odd byte offsets of the user input
    ("ring", 5, 4, 70001, "int8", "max", 1 << 17),
    ("nhr", 2, 3, 64, "fp32", "prod", 1 << 20),
    ("nb", 2, 16, 4099, "int16", "sum", 1 << 19),
    ("ring", 4, 8, 5000, "int32", "min", 1 << 20),
    ("nhr", 7, 4, 9, "int32", "sum", 28 * 128),         # second shares empty
    ("nb", 5, 3, 30011, "bf16", "sum", 1 << 18),
    ("ring", 2, 3, 0, "fp32", "sum", 4096),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


# level-1 and level-2 algorithm, pods, servers per pod, devices per server, elements per block, dtype, op, CCL buffer bytes
POD_CASES = [
    ("ring", "ring", 2, 2, 8, 1 << 16, "bf16", "sum", 8 << 20),
    ("nhr", "nb", 3, 2, 4, 50021, "fp32", "sum", 1 << 21),
    ("nb", "nhr", 2, 3, 5, 30011, "fp16", "max", 1 << 19),
    ("ring", "nhr", 4, 1, 8, 4099, "int16", "sum", 1 << 19),
    ("nhr", "ring", 2, 5, 3, 777, "int8", "min", 30 * 128),
    ("ring", "nb", 5, 2, 3, 64, "fp32", "prod", 1 << 20),
]


def run_case(thread, alg, n_servers, n_local, count, dtype, op, ccl, seed=0, n_pods=1, alg2="ring"):
    dt, o, n = DT[dtype], OPS[op], n_pods * n_servers * n_local
    host_in = [gen(dt, n * count, 16000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 994, "wide")
    junk = np.random.default_rng(17).integers(0, 256, ccl, dtype=np.uint8)
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [junk.copy() for _ in range(n)]
    oracle.run_dbring_rs_servers(ALG[alg], n_servers, n_local, w_in, w_out, w_cin, count, ccl, dt, o, n_pods=n_pods, alg2=ALG[alg2])
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cin = [to_dev(junk) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptrs = lambda ts: [t.data_ptr() if t.numel() else pad.data_ptr() for t in ts]
    plan = h.DoubleRingHierReduceScatterPlan(ALG[alg], n_servers, n_local, ptrs(d_in), ptrs(d_out), ptrs(d_cin), ccl, count, dt, o,
                                             n_pods=n_pods, alg2=ALG[alg2])
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "user out[%d]" % r)
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cin[r], junk), w_cin[r]), "CCL in[%d]" % r
        ops = oracle.trace_dbring_rs_servers(ALG[alg], n_servers, n_local, count, ccl, dt, n_pods=n_pods, alg2=ALG[alg2])
        assert plan.info.algorithmicBytes == sum(x[8] * (3 if x[1] else 2) for x in ops)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("alg,n_servers,n_local,count,dtype,op,ccl", CASES)
def test_double_ring_reduce_scatter_over_servers_matches_oracle(gpu_thread, alg, n_servers, n_local, count, dtype, op, ccl):
    say("double ring rs over servers", alg, n_servers, n_local, count, dtype, op, ccl)
    run_case(gpu_thread, alg, n_servers, n_local, count, dtype, op, ccl)


@pytest.mark.parametrize("alg,alg2,n_pods,n_servers,n_local,count,dtype,op,ccl", POD_CASES)
def test_double_ring_reduce_scatter_over_pods_matches_oracle(gpu_thread, alg, alg2, n_pods, n_servers, n_local, count, dtype, op, ccl):
    say("double ring rs over pods", alg, alg2, n_pods, n_servers, n_local, count, dtype, op, ccl)
    run_case(gpu_thread, alg, n_servers, n_local, count, dtype, op, ccl, n_pods=n_pods, alg2=alg2)


def test_launch_count(gpu_thread):
    """2 x 8 ranks, one chunk: the 128 fetches of the init step in two launches (a launch carries at most 64 segments),
    then per ring step one reduce and one copy launch of 64 segments each (the last without copies), the fold between
    the two servers and the copy out."""
    info = run_case(gpu_thread, "ring", 2, 8, 1 << 16, "bf16", "sum", 4 << 20)
    assert info.launches == 2 + 6 * 2 + 1 + 1 + 1


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(8282)
    for i in range(30):
        n_local = int(rng.integers(3, 9))
        n_pods = int(rng.integers(1, 3))
        n_servers = int(rng.integers(3 - n_pods, 32 // (n_local * n_pods) + 1))
        count = int(rng.integers(1, 60000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        alg = ["ring", "nhr", "nb"][rng.integers(3)]
        alg2 = ["ring", "nhr", "nb"][rng.integers(3)]
        ccl = int(rng.integers(1, 64)) * 128 * n_pods * n_servers * n_local * 4
        say("random double ring rs over servers", i, alg, alg2, n_pods, n_servers, n_local, count, dtype, op, ccl)
        run_case(gpu_thread, alg, n_servers, n_local, count, dtype, op, ccl, seed=i, n_pods=n_pods, alg2=alg2)
