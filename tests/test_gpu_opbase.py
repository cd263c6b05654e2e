"""GPU parity of the op-base loop plans (user buffers -> CCL buffers -> template -> user buffers) against the CPU
oracle's transcription of the executors' loop: after the run the user outputs, the untouched user inputs and
what is left in the CCL and communication buffers are compared bit for bit."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

ALGS = {
    "ring_ar": oracle.ALG_ALLREDUCE_RING, "rhd_ar": oracle.ALG_ALLREDUCE_RHD, "mesh_oneshot": oracle.ALG_ALLREDUCE_MESH_ONESHOT,
    "nhr_ar": oracle.ALG_ALLREDUCE_NHR, "nb_ar": oracle.ALG_ALLREDUCE_NB, "chunk_mesh": oracle.ALG_ALLREDUCE_CHUNK_MESH,
    "local_reduce": oracle.ALG_ALLREDUCE_LOCAL_REDUCE, "mesh_rs": oracle.ALG_RS_MESH, "ring_rs": oracle.ALG_RS_RING_STANDALONE,
    "nhr_rs": oracle.ALG_RS_NHR, "nb_rs": oracle.ALG_RS_NB, "local_reduce_rs": oracle.ALG_RS_LOCAL_REDUCE,
    "doubling": oracle.ALG_ALLREDUCE_DOUBLING, "nhr_oneshot": oracle.ALG_ALLREDUCE_NHR_ONESHOT,
}
SCATTER = {"mesh_rs", "ring_rs", "nhr_rs", "nb_rs", "local_reduce_rs"}
NOT_FUSABLE = {"chunk_mesh", "local_reduce", "local_reduce_rs", "doubling"}

# algorithm, ranks, elements, dtype, op, CCL buffer bytes
CASES = [
    ("ring_ar", 8, 1 << 20, "bf16", "sum", 8 << 20),       # one pass: the message fits the CCL buffer
    ("ring_ar", 8, 300007, "fp32", "sum", 1 << 18),        # 5 chunks, ragged last one
    ("ring_ar", 3, 70001, "int8", "max", 4096),            # 18 chunks
    ("rhd_ar", 6, 100003, "fp16", "sum", 1 << 17),
    ("mesh_oneshot", 8, 2048, "fp16", "sum", 1 << 20),
    ("nhr_ar", 5, 40009, "fp32", "min", 1 << 16),
    ("nb_ar", 7, 300007, "int32", "sum", 1 << 20),
    ("chunk_mesh", 4, 100003, "bf16", "sum", 1 << 17),
    ("local_reduce", 8, 100003, "fp32", "sum", 1 << 18),
    ("mesh_rs", 8, 40001, "fp32", "sum", 1 << 18),         # 8 x 128-byte-aligned slices of 32 KiB per chunk
    ("ring_rs", 7, 5000, "bf16", "sum", 1 << 20),          # one pass: a single copy of the whole input
    ("nhr_rs", 5, 70001, "int8", "sum", 1 << 16),
    ("nb_rs", 12, 9999, "int32", "max", 1 << 16),
    ("local_reduce_rs", 6, 50001, "fp16", "sum", 1 << 17),
    ("ring_ar", 1, 1000, "fp32", "sum", 1024),
    ("doubling", 8, 40009, "fp16", "sum", 1 << 16),
    ("nhr_oneshot", 5, 40009, "bf16", "sum", 1 << 16),
]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_case(thread, name, lowering, n, count, dtype, op, ccl):
    dt, o, alg = DT[dtype], OPS[op], ALGS[name]
    in_count = n * count if name in SCATTER else count
    host_in = [gen(dt, in_count, 4000 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, count, 998, "wide")
    junk = np.random.default_rng(11).integers(0, 256, ccl, dtype=np.uint8)
    chunk = min(count, oracle.opbase_max_count(alg, n, ccl, dt))
    sb = h.scratch_bytes(alg, n, chunk, dt)
    sjunk = np.random.default_rng(12).integers(0, 256, sb, dtype=np.uint8) if sb else None
    w_in = [x.copy() for x in host_in]
    w_out = [sentinel.copy() for _ in range(n)]
    w_cin = [junk.copy() for _ in range(n)]
    w_cout = [junk[::-1].copy() for _ in range(n)]
    w_scr = [sjunk.copy() for _ in range(n)] if sb else None
    oracle.run_opbase(alg, w_in, w_out, w_cin, w_cout, count, ccl, dt, o, scratch=w_scr)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_cin = [to_dev(junk) for _ in range(n)]
    d_cout = [to_dev(junk[::-1].copy()) for _ in range(n)]
    d_scr = [to_dev(sjunk) for _ in range(n)] if sb else None
    ptrs = lambda ts: [t.data_ptr() for t in ts]
    plan = h.OpBasePlan(alg, lowering, ptrs(d_in), ptrs(d_out), ptrs(d_cin), ptrs(d_cout), ccl, count, dt, o,
                        ptrs(d_scr) if sb else None)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], sentinel), w_out[r], dt, "%s user out[%d]" % (name, r))
            assert np.array_equal(from_dev(d_in[r], host_in[r]).view(np.uint8), host_in[r].view(np.uint8)), "user in[%d] was written" % r
            assert np.array_equal(from_dev(d_cin[r], junk), w_cin[r]), "%s CCL in[%d]" % (name, r)
            assert np.array_equal(from_dev(d_cout[r], junk), w_cout[r]), "%s CCL out[%d]" % (name, r)
            if sb:
                assert np.array_equal(from_dev(d_scr[r], sjunk), w_scr[r]), "%s scratch[%d]" % (name, r)
        assert plan.info.algorithmicBytes == oracle.algorithmic_bytes_opbase(alg, n, count, ccl, dt)
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("name,n,count,dtype,op,ccl", CASES)
def test_opbase_stepwise_matches_oracle(gpu_thread, name, n, count, dtype, op, ccl):
    say("opbase stepwise", name, n, count, dtype, op, ccl)
    info = run_case(gpu_thread, name, h.Lowering.STEPWISE, n, count, dtype, op, ccl)
    assert info.movedBytes == info.algorithmicBytes


@pytest.mark.parametrize("name,n,count,dtype,op,ccl", [c for c in CASES if c[0] not in NOT_FUSABLE])
def test_opbase_fused_leaves_identical_memory(gpu_thread, name, n, count, dtype, op, ccl):
    say("opbase fused", name, n, count, dtype, op, ccl)
    info = run_case(gpu_thread, name, h.Lowering.FUSED, n, count, dtype, op, ccl)
    assert info.movedBytes <= info.algorithmicBytes


def test_randomized_opbase_shapes(gpu_thread):
    """A fixed-seed sample of (algorithm, rank count, element count, type, CCL buffer size, lowering) through the op-base
    loop: one pass, many chunks, ragged last chunks."""
    rng = np.random.default_rng(777)
    names = sorted(ALGS)
    done = 0
    while done < 60:
        name = names[rng.integers(len(names))]
        n = int(rng.integers(1, 13))
        if name in ("local_reduce", "doubling"):
            n = 1 << int(rng.integers(0, 4))
        count = int(rng.integers(1, 60000))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min"][rng.integers(3)]
        ccl = int(rng.integers(1, 64)) * 128 * n * 4
        lowering = h.Lowering.FUSED if (name not in NOT_FUSABLE and rng.integers(2)) else h.Lowering.STEPWISE
        say("random opbase", done, name, n, count, dtype, op, ccl, lowering)
        run_case(gpu_thread, name, lowering, n, count, dtype, op, ccl)
        done += 1
