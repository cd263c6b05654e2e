"""GPU parity of the three-step allreduce plans (ring reduce-scatter inside the servers, the level-1 template between
them on the own segment, ring all-gather inside) against the CPU oracle's per-rank transcription of the ring executor:
inputs (which hold the partial sums of the first two steps) and outputs bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

LEVEL1 = {"ring": oracle.ALG_ALLREDUCE_RING, "rhd": oracle.ALG_ALLREDUCE_RHD, "nhr": oracle.ALG_ALLREDUCE_NHR,
          "nb": oracle.ALG_ALLREDUCE_NB}

# level-1 algorithm, servers, ranks per server, elements, dtype, op
CASES = [
    ("ring", 2, 8, 1 << 20, "bf16", "sum"),
    ("rhd", 4, 8, 1000003, "fp32", "sum"),
    ("nhr", 4, 8, 1 << 21, "bf16", "sum"),         # 512 KiB per device: the sliced NHR template between the servers
    ("nhr", 4, 8, 100003, "fp16", "sum"),          # small: the one-shot NHR template
    ("nb", 3, 5, 300007, "int32", "max"),
    ("rhd", 5, 3, 70001, "int8", "sum"),
    ("ring", 2, 2, 100, "fp32", "prod"),
    ("nhr", 3, 4, 3 * 70000 + 1, "fp32", "min"),
    ("ring", 1, 8, 100003, "fp32", "sum"),         # one server: reduce-scatter, a copy of the segment, all-gather
    ("rhd", 8, 1, 100003, "int16", "sum"),         # one rank per server: the level-1 template alone
    ("nb", 2, 16, 9, "int32", "sum"),              # most segments empty
    ("ring", 4, 4, 0, "fp32", "sum"),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, alg1, ns, nl, count, dtype, op, seed=0, mesh=False):
    dt, o, n = DT[dtype], OPS[op], ns * nl
    host_in = [gen(dt, count, 7000 + seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 997, "wide")
    want_in = [x.copy() for x in host_in]
    want_out = [sentinel.copy() for _ in range(n)]
    oracle.run_hier(LEVEL1[alg1], ns, nl, want_in, want_out, count, dt, o, mesh=mesh)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptr = lambda t: t.data_ptr() if t.numel() else pad.data_ptr()
    plan = h.HierPlan(LEVEL1[alg1], ns, nl, [ptr(t) for t in d_in], [ptr(t) for t in d_out], count, dt, o, mesh=mesh)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_in[r], host_in[r]), want_in[r], dt, "in[%d]" % r)
            assert_same(from_dev(d_out[r], sentinel), want_out[r], dt, "out[%d]" % r)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("alg1,ns,nl,count,dtype,op", CASES)
def test_three_step_allreduce_matches_oracle(gpu_thread, alg1, ns, nl, count, dtype, op):
    say("hier", alg1, ns, nl, count, dtype, op)
    info = run_case(gpu_thread, alg1, ns, nl, count, dtype, op)
    ops = oracle.trace_hier(LEVEL1[alg1], ns, nl, count, DT[dtype])
    assert info.algorithmicBytes == sum(o[8] * (3 if o[1] else 2) for o in ops)
    assert info.movedBytes == info.algorithmicBytes
    assert info.launches <= 2 * (max(o[0] for o in ops) + 1 if ops else 0)     # about one launch per lock-step step


@pytest.mark.parametrize("alg1,ns,nl,count,dtype,op", CASES)
def test_three_step_allreduce_with_mesh_level0_matches_oracle(gpu_thread, alg1, ns, nl, count, dtype, op):
    if nl < 2:
        pytest.skip("the mesh executor needs at least two ranks per server")
    say("mesh hier", alg1, ns, nl, count, dtype, op)
    info = run_case(gpu_thread, alg1, ns, nl, count, dtype, op, mesh=True)
    ops = oracle.trace_hier(LEVEL1[alg1], ns, nl, count, DT[dtype], mesh=True)
    assert info.algorithmicBytes == sum(o[8] * (3 if o[1] else 2) for o in ops)
    assert info.movedBytes == info.algorithmicBytes


def test_randomized_shapes(gpu_thread):
    rng = np.random.default_rng(4242)
    names = sorted(LEVEL1)
    for i in range(40):
        alg1 = names[rng.integers(len(names))]
        ns, nl = int(rng.integers(1, 9)), int(rng.integers(1, 9))
        if ns * nl > 32:
            nl = 32 // ns
        count = int(rng.integers(1, 400000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        mesh = bool(rng.integers(2)) and nl >= 2
        say("random hier", i, alg1, ns, nl, count, dtype, op, mesh)
        run_case(gpu_thread, alg1, ns, nl, count, dtype, op, seed=i, mesh=mesh)
