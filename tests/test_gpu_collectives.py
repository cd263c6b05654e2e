"""GPU parity of the schedule replays (both lowerings) against the CPU oracle: every one of the 2N rank
buffers is compared bit-for-bit after the run, so intermediate partials left in the input buffers count."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, UNIT, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu

ALGS = {
    "ring_ar": (h.Alg.ALLREDUCE_RING, oracle.ALG_ALLREDUCE_RING),
    "ring_rs_stage": (h.Alg.REDUCE_SCATTER_RING, oracle.ALG_RS_RING_STAGE),
    "rhd_ar": (h.Alg.ALLREDUCE_RHD, oracle.ALG_ALLREDUCE_RHD),
    "mesh_oneshot": (h.Alg.ALLREDUCE_MESH_ONESHOT, oracle.ALG_ALLREDUCE_MESH_ONESHOT),
    "mesh_rs": (h.Alg.REDUCE_SCATTER_MESH, oracle.ALG_RS_MESH),
    "ring_rs": (h.Alg.REDUCE_SCATTER_RING_STANDALONE, oracle.ALG_RS_RING_STANDALONE),
    "mesh_ascending": (h.Alg.ALLREDUCE_MESH_ONESHOT_ASCENDING, oracle.ALG_ALLREDUCE_MESH_ASCENDING),
    "local_reduce": (h.Alg.ALLREDUCE_LOCAL_REDUCE, oracle.ALG_ALLREDUCE_LOCAL_REDUCE),
    "chunk_mesh": (h.Alg.ALLREDUCE_CHUNK_MESH, oracle.ALG_ALLREDUCE_CHUNK_MESH),
    "nhr_ar": (h.Alg.ALLREDUCE_NHR, oracle.ALG_ALLREDUCE_NHR),
    "nhr_rs": (h.Alg.REDUCE_SCATTER_NHR, oracle.ALG_RS_NHR),
    "nb_ar": (h.Alg.ALLREDUCE_NB, oracle.ALG_ALLREDUCE_NB),
    "nb_rs": (h.Alg.REDUCE_SCATTER_NB, oracle.ALG_RS_NB),
    "local_reduce_rs": (h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, oracle.ALG_RS_LOCAL_REDUCE),
    "doubling": (h.Alg.ALLREDUCE_DOUBLING, oracle.ALG_ALLREDUCE_DOUBLING),
    "nhr_oneshot": (h.Alg.ALLREDUCE_NHR_ONESHOT, oracle.ALG_ALLREDUCE_NHR_ONESHOT),
    "window_rs": (h.Alg.REDUCE_SCATTER_WINDOW_HALVING, oracle.ALG_RS_WINDOW_HALVING),
}
SCATTER = ("mesh_rs", "ring_rs", "nhr_rs", "nb_rs", "window_rs")
FUSABLE = {"ring_ar", "ring_rs_stage", "rhd_ar", "mesh_oneshot", "mesh_rs", "ring_rs", "mesh_ascending",
           "nhr_ar", "nhr_rs", "nb_ar", "nb_rs", "nhr_oneshot"}
# fused onto the user buffers alone: the communication buffers are not touched, only the inputs and outputs compare
FUSABLE_NO_SCRATCH = {"window_rs"}


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def buffer_counts(alg, n, count, stride=0):
    """(elements in each input buffer, elements in each output buffer)."""
    if alg in SCATTER or alg == "local_reduce_rs":
        return ((n - 1) * stride + count if stride else n * count), count
    return count, count


def run_case(thread, alg, lowering, n, count, dtype, op, seed=0, kind=None, stride=0):
    dt, o = DT[dtype], OPS[op]
    in_count, out_count = buffer_counts(alg, n, count, stride)
    kind = kind or ("prod" if op == "prod" else "default")
    host_in = [gen(dt, in_count, seed * 1000 + r, kind) for r in range(n)]
    sentinel = gen(dt, out_count, 999, "wide")
    want_in = [x.copy() for x in host_in]
    want_out = [sentinel.copy() for _ in range(n)]
    sb = h.scratch_bytes(ALGS[alg][0], n, count, dt)
    junk = np.random.default_rng(5).integers(0, 256, sb, dtype=np.uint8) if sb else None
    want_scr = [junk.copy() for _ in range(n)] if sb else None
    oracle.run(ALGS[alg][1], want_in, want_out, count, dt, o, stride, scratch=want_scr)
    # every device buffer carries 64 guard bytes behind its last element: a kernel that runs past a buffer's end
    # (a tail handled by the wrong tile, a workgroup of a wider grid that should have found nothing to do) shows there
    guard = np.arange(64, dtype=np.uint8) ^ 0xA5
    up = lambda a: to_dev(np.concatenate([np.ascontiguousarray(a).view(np.uint8).ravel(), guard]))
    body = lambda t, like: t[:like.nbytes].cpu().numpy().view(like.dtype).reshape(like.shape)
    tail = lambda t, like: t[like.nbytes:].cpu().numpy()
    d_in = [up(x) for x in host_in]
    d_out = [up(sentinel) for _ in range(n)]
    d_scr = [up(junk) for _ in range(n)] if sb else None
    plan = h.Plan(ALGS[alg][0], lowering, [t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out], count, dt, o, stride,
                  [t.data_ptr() for t in d_scr] if sb else None)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        for r in range(n):
            assert_same(body(d_in[r], host_in[r]), want_in[r], dt, "in[%d]" % r)
            assert_same(body(d_out[r], sentinel), want_out[r], dt, "out[%d]" % r)
            assert np.array_equal(tail(d_in[r], host_in[r]), guard), "bytes behind in[%d] written" % r
            assert np.array_equal(tail(d_out[r], sentinel), guard), "bytes behind out[%d] written" % r
            if sb and lowering == h.Lowering.STEPWISE:  # the communication buffer too (bytes never written keep their junk)
                assert np.array_equal(body(d_scr[r], junk), want_scr[r]), "scratch[%d]" % r
                assert np.array_equal(tail(d_scr[r], junk), guard), "bytes behind scratch[%d] written" % r
        return plan.info.launches, plan.info.algorithmicBytes, plan.info.movedBytes
    finally:
        plan.destroy()


CASES = [
    # alg, n, count, dtype, op
    ("ring_ar", 8, 1 << 20, "fp32", "sum"),        # benchmark config 1
    ("ring_ar", 8, 1000003, "bf16", "sum"),
    ("ring_ar", 7, 100003, "fp16", "sum"),
    ("ring_ar", 3, 5, "int8", "sum"),              # most slices empty
    ("ring_ar", 2, 4099, "int32", "max"),
    ("ring_ar", 1, 777, "fp32", "sum"),
    ("ring_ar", 5, 0, "fp32", "sum"),
    ("ring_ar", 16, 70001, "int16", "min"),
    ("ring_ar", 32, 300007, "bf16", "max"),
    ("ring_ar", 4, 65536, "fp32", "prod"),
    ("ring_rs_stage", 7, 1000003, "fp32", "prod"),  # benchmark config 5a, scaled down
    ("ring_rs_stage", 7, 1000003, "int8", "sum"),   # benchmark config 5b, scaled down (odd last slice)
    ("ring_rs_stage", 8, 123457, "bf16", "sum"),
    ("rhd_ar", 16, 1 << 18, "int32", "sum"),       # benchmark config 3, scaled down
    ("rhd_ar", 16, 1 << 18, "int32", "max"),
    ("rhd_ar", 16, 1 << 18, "int32", "min"),
    ("rhd_ar", 8, 100003, "fp32", "sum"),
    ("rhd_ar", 6, 100003, "fp16", "sum"),          # part one: ranks 0..3 fold in pairs
    ("rhd_ar", 7, 50001, "bf16", "sum"),
    ("rhd_ar", 5, 33, "int8", "sum"),
    ("rhd_ar", 3, 1 << 16, "fp32", "max"),
    ("rhd_ar", 2, 12345, "int16", "sum"),
    ("rhd_ar", 1, 100, "int32", "sum"),
    ("rhd_ar", 12, 77777, "fp32", "sum"),
    ("rhd_ar", 32, 100003, "bf16", "sum"),
    ("rhd_ar", 31, 4099, "int16", "max"),
    ("rhd_ar", 17, 100003, "fp32", "min"),
    ("rhd_ar", 4, 65536, "fp32", "prod"),
    ("mesh_oneshot", 8, 2048, "fp16", "sum"),      # benchmark config 4, 4 KiB
    ("mesh_oneshot", 8, 1 << 21, "fp16", "sum"),   # benchmark config 4, 4 MiB
    ("mesh_oneshot", 8, 100003, "fp32", "sum"),
    ("mesh_oneshot", 5, 4097, "bf16", "max"),
    ("mesh_oneshot", 2, 1, "int8", "sum"),
    ("mesh_oneshot", 1, 1000, "fp32", "sum"),
    ("mesh_rs", 8, 40001, "fp32", "sum"),
    ("mesh_rs", 4, 4096, "fp16", "min"),
    ("mesh_rs", 7, 999, "int32", "sum"),
    ("ring_rs", 8, 40001, "fp32", "sum"),
    ("ring_rs", 7, 5000, "bf16", "sum"),
    ("ring_rs", 2, 64, "int8", "max"),
    ("mesh_ascending", 8, 100003, "fp16", "sum"),
    ("mesh_ascending", 5, 4097, "fp32", "max"),
    ("mesh_ascending", 1, 10, "int8", "sum"),
    ("local_reduce", 8, 1 << 20, "bf16", "sum"),
    ("local_reduce", 4, 100003, "fp32", "sum"),
    ("local_reduce", 16, 70001, "fp16", "max"),
    ("local_reduce", 32, 300007, "int32", "sum"),
    ("local_reduce", 2, 4099, "int8", "min"),
    ("local_reduce", 8, 1001, "int16", "sum"),     # slots fall back to 512-byte / element alignment
    ("local_reduce", 8, 7, "fp32", "sum"),
    ("local_reduce", 1, 100, "fp32", "sum"),
    ("local_reduce", 3, 100003, "fp32", "sum"),    # the one rank count besides the powers of two whose folds land
    ("local_reduce", 3, 5, "bf16", "max"),
    ("chunk_mesh", 8, 1 << 20, "bf16", "sum"),
    ("chunk_mesh", 7, 100003, "fp32", "sum"),
    ("chunk_mesh", 3, 4099, "fp16", "max"),
    ("chunk_mesh", 2, 70001, "int8", "sum"),
    ("chunk_mesh", 16, 300007, "int32", "min"),
    ("chunk_mesh", 5, 9, "int16", "sum"),
    ("chunk_mesh", 1, 100, "fp32", "sum"),
    ("nhr_ar", 8, 1 << 20, "bf16", "sum"),
    ("nhr_ar", 7, 100003, "fp32", "sum"),
    ("nhr_ar", 5, 4099, "fp16", "max"),            # step 0 of rank 0 folds two slices that do not touch
    ("nhr_ar", 3, 70001, "int8", "sum"),
    ("nhr_ar", 16, 300007, "int32", "min"),
    ("nhr_ar", 31, 4099, "int16", "max"),
    ("nhr_ar", 12, 1000, "fp32", "prod"),
    ("nhr_ar", 2, 9, "bf16", "sum"),
    ("nhr_ar", 1, 100, "fp32", "sum"),
    ("nhr_rs", 8, 40001, "fp32", "sum"),
    ("nhr_rs", 7, 5000, "bf16", "sum"),
    ("nhr_rs", 5, 64, "int8", "max"),
    ("nhr_rs", 32, 1001, "int32", "sum"),           # 16 unmerged slices per rank at step 0: several launches
    ("nb_ar", 8, 1 << 20, "bf16", "sum"),
    ("nb_ar", 7, 100003, "fp32", "sum"),            # below 128 KiB per rank: cut in 128 KiB granules, not in 7
    ("nb_ar", 6, 300007, "int32", "min"),
    ("nb_ar", 16, 1 << 21, "fp16", "max"),
    ("nb_ar", 3, 70001, "int8", "sum"),
    ("nb_ar", 1, 100, "fp32", "sum"),
    ("nb_rs", 8, 40001, "fp32", "sum"),
    ("nb_rs", 7, 5000, "bf16", "sum"),
    ("nb_rs", 12, 999, "int32", "sum"),
    ("local_reduce_rs", 8, 1 << 20, "bf16", "sum"),
    ("local_reduce_rs", 7, 100003, "fp32", "sum"),  # receive windows start at i*400012 mod 16384: 4-byte aligned only
    ("local_reduce_rs", 6, 16384, "fp16", "max"),
    ("local_reduce_rs", 5, 70001, "int8", "sum"),   # odd byte offsets
    ("local_reduce_rs", 16, 40000, "int32", "min"),
    ("local_reduce_rs", 3, 1001, "int16", "sum"),   # up to 32 KiB: windows not staggered
    ("local_reduce_rs", 2, 9, "fp32", "prod"),
    ("local_reduce_rs", 1, 100, "fp32", "sum"),
    ("doubling", 8, 2048, "fp16", "sum"),           # its use: small messages inside a server
    ("doubling", 16, 100003, "fp32", "max"),
    ("doubling", 4, 1 << 20, "bf16", "sum"),
    ("doubling", 2, 9, "int8", "min"),
    ("doubling", 1, 100, "int32", "sum"),
    ("nhr_oneshot", 8, 65536, "bf16", "sum"),       # its use: messages the NHR allreduce does not slice
    ("nhr_oneshot", 5, 100003, "fp32", "sum"),
    ("nhr_oneshot", 13, 4099, "fp16", "max"),
    ("nhr_oneshot", 32, 70001, "int16", "min"),
    ("nhr_oneshot", 2, 9, "int8", "sum"),
    ("nhr_oneshot", 3, 1 << 20, "fp32", "prod"),
    ("nhr_oneshot", 1, 100, "int32", "sum"),
    ("nhr_oneshot", 6, 0, "fp32", "sum"),
    ("window_rs", 8, 1 << 18, "bf16", "sum"),       # the AICPU deterministic reduce-scatter: whole windows folded in halves
    ("window_rs", 7, 100003, "fp32", "sum"),        # 3 slots beyond the largest power of two, odd block sizes
    ("window_rs", 6, 16384, "fp16", "max"),
    ("window_rs", 5, 70001, "int8", "sum"),
    ("window_rs", 3, 1001, "int16", "sum"),
    ("window_rs", 2, 9, "fp32", "prod"),
    ("window_rs", 1, 100, "fp32", "sum"),
    ("window_rs", 12, 4104, "fp16", "sum"),
    ("window_rs", 32, 8200, "fp32", "min"),
    ("window_rs", 4, 0, "fp32", "sum"),
]


@pytest.mark.parametrize("alg,n,count,dtype,op", CASES)
def test_stepwise_replay_matches_oracle(gpu_thread, alg, n, count, dtype, op):
    say("stepwise", alg, n, count, dtype, op)
    launches, algo, moved = run_case(gpu_thread, alg, h.Lowering.STEPWISE, n, count, dtype, op)
    assert algo == oracle.algorithmic_bytes(ALGS[alg][1], n, count, DT[dtype])
    assert moved == algo, "the step-wise lowering moves exactly the two-input model's bytes"


@pytest.mark.parametrize("alg,n,count,dtype,op", [c for c in CASES if c[0] in FUSABLE]
                         + [c for c in CASES if c[0] in FUSABLE_NO_SCRATCH and (c[2] * UNIT[DT[c[3]]]) % 16 == 0])
def test_fused_lowering_leaves_identical_memory(gpu_thread, alg, n, count, dtype, op):
    say("fused", alg, n, count, dtype, op)
    launches, algo, moved = run_case(gpu_thread, alg, h.Lowering.FUSED, n, count, dtype, op)
    assert launches <= 1
    assert moved <= algo


USER_BUFFER_FUSED = [
    # alg, n, count, dtype, op: single-launch lowerings that leave the communication buffers alone
    ("local_reduce_rs", 8, 1 << 20, "bf16", "sum"), ("local_reduce_rs", 7, 100004, "fp32", "sum"),
    ("local_reduce_rs", 6, 16384, "fp16", "max"), ("local_reduce_rs", 5, 70016, "int8", "sum"),
    ("local_reduce_rs", 16, 40000, "int32", "min"), ("local_reduce_rs", 3, 1000, "int16", "sum"),
    ("local_reduce_rs", 2, 8, "fp32", "prod"), ("local_reduce_rs", 1, 100, "fp32", "sum"),
    ("local_reduce_rs", 12, 4104, "fp16", "sum"), ("local_reduce_rs", 31, 4096, "bf16", "max"),
    ("local_reduce_rs", 32, 8200, "fp32", "sum"), ("local_reduce_rs", 4, 0, "fp32", "sum"),
    ("chunk_mesh", 8, 1 << 20, "bf16", "sum"), ("chunk_mesh", 7, 100003, "fp32", "sum"),
    ("chunk_mesh", 6, 16385, "fp16", "max"), ("chunk_mesh", 5, 70001, "int8", "sum"),
    ("chunk_mesh", 16, 400007, "int32", "min"), ("chunk_mesh", 3, 1001, "int16", "sum"),
    ("chunk_mesh", 2, 9, "fp32", "prod"), ("chunk_mesh", 1, 100, "fp32", "sum"), ("chunk_mesh", 4, 0, "fp32", "sum"),
    ("chunk_mesh", 12, 77777, "fp16", "sum"), ("chunk_mesh", 31, 300007, "bf16", "max"),
    ("chunk_mesh", 32, 1 << 20, "fp32", "sum"), ("chunk_mesh", 8, 100, "fp32", "sum"),  # most sub-chunks empty
    ("local_reduce", 8, 1 << 20, "bf16", "sum"), ("local_reduce", 4, 100003, "fp32", "sum"),
    ("local_reduce", 16, 70001 * 16, "fp16", "max"), ("local_reduce", 2, 4099, "int8", "sum"),
    ("local_reduce", 8, 300007, "int32", "min"), ("local_reduce", 4, 65536, "fp32", "prod"),
    ("local_reduce", 16, 1 << 20, "bf16", "sum"), ("local_reduce", 8, 8 * 8192 + 24, "int16", "sum"),
    ("local_reduce", 1, 100, "fp32", "sum"), ("local_reduce", 4, 0, "fp32", "sum"),
    ("local_reduce", 3, 100003, "fp32", "sum"), ("local_reduce", 3, 3 * 8192 + 8, "fp16", "min"),
    ("local_reduce", 32, 1 << 20, "bf16", "sum"), ("local_reduce", 32, 32 * 4096 + 100, "fp32", "max"),  # trees of depth 6
    ("window_rs", 8, 1 << 20, "bf16", "sum"), ("window_rs", 7, 100004, "fp32", "sum"), ("window_rs", 6, 16384, "fp16", "max"),
    ("window_rs", 5, 70016, "int8", "sum"), ("window_rs", 3, 1000, "int16", "sum"), ("window_rs", 2, 8, "fp32", "prod"),
    ("window_rs", 1, 100, "fp32", "sum"), ("window_rs", 12, 4104, "fp16", "sum"), ("window_rs", 31, 4096, "bf16", "max"),
    ("window_rs", 32, 8200, "fp32", "sum"), ("window_rs", 4, 0, "fp32", "sum"),
]


@pytest.mark.parametrize("alg,n,count,dtype,op", USER_BUFFER_FUSED)
def test_fused_lowerings_on_the_user_buffers(gpu_thread, alg, n, count, dtype, op):
    """One tree launch in place of the deterministic reduce-scatter's slot writes and halving rounds, one chain
    launch per group of ranks in place of the chunk-mesh allreduce's rounds and gather, tree launches laid out from the
    deterministic allreduce's own operation list: the user outputs hold the oracle's bits, the inputs are only read,
    and no communication buffer is asked for."""
    say("fused on user buffers", alg, n, count, dtype, op)
    dt, o = DT[dtype], OPS[op]
    in_count, out_count = buffer_counts(alg, n, count)
    host_in = [gen(dt, in_count, 7000 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, out_count, 999, "wide")
    want_in = [x.copy() for x in host_in]
    want_out = [sentinel.copy() for _ in range(n)]
    sb = h.scratch_bytes(ALGS[alg][0], n, count, dt)
    oracle.run(ALGS[alg][1], want_in, want_out, count, dt, o,
               scratch=[np.zeros(sb, np.uint8) for _ in range(n)] if sb else None)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptr = lambda t: t.data_ptr() if t.numel() else pad.data_ptr()
    plan = h.Plan(ALGS[alg][0], h.Lowering.FUSED, [ptr(t) for t in d_in], [ptr(t) for t in d_out], count, dt, o)
    try:
        unit = host_in[0].itemsize
        if alg in ("local_reduce_rs", "window_rs"):
            assert plan.info.launches == (1 if count else 0)
            if n > 1:
                assert plan.info.movedBytes == (n + 1) * n * count * unit
        elif n > 1:
            per_launch = 32 // (n - 1) if alg == "chunk_mesh" else 8   # segments a launch's tables hold
            if alg == "local_reduce" and n > 16:
                per_launch = 4                                         # trees over 64 leaf positions: 256 table bytes / 64
            assert plan.info.launches <= -(-n // per_launch)
            assert plan.info.movedBytes == 2 * n * count * unit
        for rec in plan.launches():
            assert rec.kind == (h.Kernel.COPY if n == 1 else h.Kernel.CHAIN if alg == "chunk_mesh" else h.Kernel.TREE)
        assert plan.run(gpu_thread) == 0
        assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
        for r in range(n):
            assert_same(from_dev(d_in[r], host_in[r]), host_in[r], dt, "in[%d]" % r)
            assert_same(from_dev(d_out[r], sentinel), want_out[r], dt, "out[%d]" % r)
    finally:
        plan.destroy()


def test_fused_deterministic_reduce_scatter_needs_16_byte_slices():
    with pytest.raises(h.HcommError) as e:
        h.Plan(h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, h.Lowering.FUSED, [4096 * (r + 1) for r in range(4)],
               [4096 * (r + 9) for r in range(4)], 100003, DT["fp32"], OPS["sum"])
    assert e.value.code == h.HcclResult.E_NOT_SUPPORT


KEEP_INPUTS = ([c for c in CASES if c[0] in FUSABLE and c[0] != "ring_rs_stage"] + [c for c in USER_BUFFER_FUSED]
               + [c for c in CASES if c[0] == "doubling"]
               + [("doubling", 32, 70001, "bf16", "sum"), ("doubling", 16, 1 << 18, "fp16", "max"), ("doubling", 2, 3, "fp32", "sum")])


@pytest.mark.parametrize("alg,n,count,dtype,op", KEEP_INPUTS)
def test_fused_lowering_that_keeps_the_inputs(gpu_thread, alg, n, count, dtype, op):
    """HCOMM_GFX_LOWER_FUSED_KEEP_INPUTS: the outputs hold the oracle's bits, the inputs are exactly what they were,
    and the launches move one read per input element and one write per output element."""
    say("keep inputs", alg, n, count, dtype, op)
    dt, o = DT[dtype], OPS[op]
    in_count, out_count = buffer_counts(alg, n, count)
    host_in = [gen(dt, in_count, 8000 + r, "prod" if op == "prod" else "default") for r in range(n)]
    sentinel = gen(dt, out_count, 999, "wide")
    want_in = [x.copy() for x in host_in]
    want_out = [sentinel.copy() for _ in range(n)]
    sb = h.scratch_bytes(ALGS[alg][0], n, count, dt)
    oracle.run(ALGS[alg][1], want_in, want_out, count, dt, o,
               scratch=[np.zeros(sb, np.uint8) for _ in range(n)] if sb else None)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    pad = to_dev(np.zeros(256, np.uint8))
    ptr = lambda t: t.data_ptr() if t.numel() else pad.data_ptr()
    plan = h.Plan(ALGS[alg][0], h.Lowering.FUSED_KEEP_INPUTS, [ptr(t) for t in d_in], [ptr(t) for t in d_out], count, dt, o)
    try:
        if alg != "doubling":   # whose steps write the inputs: no lowering that reproduces them in one launch
            fused = h.Plan(ALGS[alg][0], h.Lowering.FUSED, [ptr(t) for t in d_in], [ptr(t) for t in d_out], count, dt, o)
            assert plan.info.launches == fused.info.launches and plan.info.movedBytes <= fused.info.movedBytes
            fused.destroy()
        assert plan.run(gpu_thread) == 0
        assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
        for r in range(n):
            assert_same(from_dev(d_in[r], host_in[r]), host_in[r], dt, "in[%d]" % r)
            assert_same(from_dev(d_out[r], sentinel), want_out[r], dt, "out[%d]" % r)
    finally:
        plan.destroy()


@pytest.mark.parametrize("alg,n,count,dtype,op", [
    ("ring_ar", 6, 100003, "fp32", "sum"), ("ring_ar", 4, 65536, "bf16", "max"), ("ring_ar", 2, 5, "int8", "sum"),
    ("mesh_oneshot", 6, 4097, "fp16", "sum"), ("mesh_ascending", 5, 100003, "fp32", "sum"),
    ("local_reduce", 16, 1 << 20, "bf16", "sum"), ("doubling", 8, 2048, "fp16", "sum"),
    ("nhr_oneshot", 7, 70001, "fp32", "sum"), ("nb_ar", 6, 300007, "int32", "min"),
])
def test_op_list_as_tree_launches_that_keep_the_inputs(gpu_thread, alg, n, count, dtype, op):
    """HcommGfxPlanCreateFromOpsKeepInputs on the oracle's own operation list: outputs as the oracle's replay leaves
    them, inputs as they were."""
    say("op list as trees", alg, n, count, dtype, op)
    dt, o = DT[dtype], OPS[op]
    host_in = [gen(dt, count, 9000 + r) for r in range(n)]
    sentinel = gen(dt, count, 999, "wide")
    want_in = [x.copy() for x in host_in]
    want_out = [sentinel.copy() for _ in range(n)]
    sb = h.scratch_bytes(ALGS[alg][0], n, count, dt)
    oracle.run(ALGS[alg][1], want_in, want_out, count, dt, o,
               scratch=[np.zeros(sb, np.uint8) for _ in range(n)] if sb else None)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    plan = h.OpListKeepInputsPlan(oracle.trace(ALGS[alg][1], n, count, dt), [t.data_ptr() for t in d_in],
                                  [t.data_ptr() for t in d_out], dt, o)
    try:
        assert all(r.kind == h.Kernel.TREE for r in plan.launches())
        assert plan.run(gpu_thread) == 0
        assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
        for r in range(n):
            assert_same(from_dev(d_in[r], host_in[r]), host_in[r], dt, "in[%d]" % r)
            assert_same(from_dev(d_out[r], sentinel), want_out[r], dt, "out[%d]" % r)
    finally:
        plan.destroy()


@pytest.mark.parametrize("alg", SCATTER)
@pytest.mark.parametrize("lowering", [h.Lowering.STEPWISE, h.Lowering.FUSED])
def test_strided_reduce_scatter(gpu_thread, alg, lowering):
    """Input slices spaced strideLen elements apart (aicpu_reduce_scatter.cc:78-80); the gaps keep their bytes."""
    if lowering == h.Lowering.FUSED and alg not in FUSABLE and alg not in FUSABLE_NO_SCRATCH:
        pytest.skip("step-wise lowering only")
    for n, count, stride, dtype in ((7, 5000, 5000 + 37, "bf16"), (4, 1 << 16, 3 << 16, "fp32"), (3, 33, 64, "int8")):
        if lowering == h.Lowering.FUSED and alg in FUSABLE_NO_SCRATCH and (stride * UNIT[DT[dtype]]) % 16:
            continue  # its single launch reads block d of every input at d * stride with 128-bit accesses
        say("strided", alg, lowering, n, count, stride, dtype)
        run_case(gpu_thread, alg, lowering, n, count, dtype, "sum", stride=stride)


def test_non_associative_inputs_expose_order(gpu_thread):
    """fp32 values for which (a+b)+c != a+(b+c): a replay in any other association order fails here."""
    n, count = 4, 4096
    base = np.array([1e8, 1.0, -1e8, 1.0], np.float32)
    for alg in ("ring_ar", "rhd_ar", "mesh_oneshot", "nhr_ar", "nb_ar", "nhr_oneshot"):
        for lowering in ((h.Lowering.STEPWISE, h.Lowering.FUSED) if alg in FUSABLE else (h.Lowering.STEPWISE,)):
            host_in = [np.full(count, base[(r + i) % 4], np.float32) for i, r in enumerate(range(n))]
            for r in range(n):
                host_in[r][1::2] = base[(r + 1) % 4]
            want_in = [x.copy() for x in host_in]
            want_out = [np.zeros(count, np.float32) for _ in range(n)]
            oracle.run(ALGS[alg][1], want_in, want_out, count, oracle.F32, oracle.SUM)
            d_in = [to_dev(x) for x in host_in]
            d_out = [to_dev(np.zeros(count, np.float32)) for _ in range(n)]
            plan = h.Plan(ALGS[alg][0], lowering, [t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out], count,
                          oracle.F32, oracle.SUM)
            assert plan.run(gpu_thread) == 0
            h.HcommGfxThreadSynchronize(gpu_thread)
            for r in range(n):
                assert_same(from_dev(d_out[r], host_in[r]), want_out[r], oracle.F32, "%s out[%d]" % (alg, r))
            plan.destroy()


def test_plan_can_run_repeatedly_and_by_range(gpu_thread):
    """A plan is reusable: re-uploading inputs and running again gives the same result; RunRange over all
    launches one at a time equals Run.  From the fourth attempt on Run replays the 15 launches as a HIP graph:
    several replays, with eager work and synchronisation in between, are checked against the same result as
    the kernel-by-kernel runs."""
    n, count, dt = 8, 100003, oracle.F32
    host_in = [gen(dt, count, 50 + r) for r in range(n)]
    want_in = [x.copy() for x in host_in]
    want_out = [np.zeros(count, np.float32) for _ in range(n)]
    oracle.run(oracle.ALG_ALLREDUCE_RING, want_in, want_out, count, dt, oracle.SUM)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(np.zeros(count, np.float32)) for _ in range(n)]
    plan = h.Plan(h.Alg.ALLREDUCE_RING, h.Lowering.STEPWISE, [t.data_ptr() for t in d_in],
                  [t.data_ptr() for t in d_out], count, dt, oracle.SUM)
    import torch
    for attempt in range(8):
        for r in range(n):
            d_in[r].copy_(torch.from_numpy(host_in[r].view(np.uint8)))
            d_out[r].zero_()
        torch.cuda.synchronize()
        if attempt == 3:
            assert plan.set_graph_replay(True) == 0
        if attempt in (2, 7):
            for i in range(plan.info.launches):
                assert plan.run_range(gpu_thread, i, 1) == 0
        else:
            assert plan.run(gpu_thread) == 0
        h.HcommGfxThreadSynchronize(gpu_thread)
        for r in range(n):
            assert_same(from_dev(d_out[r], host_in[r]), want_out[r], dt)
            assert_same(from_dev(d_in[r], host_in[r]), want_in[r], dt)
    assert plan.run_range(gpu_thread, plan.info.launches, 1) == h.HcclResult.E_PARA
    plan.destroy()


def test_ring_via_public_primitives_in_batch_mode(gpu_thread):
    """Replay the oracle's op list through HcommLocalCopy/ReduceOnThread with one BatchModeStart/End per
    step - the way an external operator library would drive the data plane - and get one launch per step."""
    n, count, dt = 8, 65539, oracle.BF16
    host_in = [gen(dt, count, 70 + r) for r in range(n)]
    want_in = [x.copy() for x in host_in]
    want_out = [np.zeros(count, np.uint16) for _ in range(n)]
    oracle.run(oracle.ALG_ALLREDUCE_RING, want_in, want_out, count, dt, oracle.SUM)
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(np.zeros(count, np.uint16)) for _ in range(n)]
    bufs = (d_in, d_out)
    ops = oracle.trace(oracle.ALG_ALLREDUCE_RING, n, count, dt)
    h.HcommGfxThreadSynchronize(gpu_thread)
    h.HcommGfxLaunchLogClear(gpu_thread)
    steps = sorted(set(o[0] for o in ops))
    for s in steps:
        assert h.HcommBatchModeStart(None) == 0
        for (step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes) in ops:
            if step != s:
                continue
            dst = bufs[dbuf][rank].data_ptr() + doff
            src = bufs[sbuf][srank].data_ptr() + soff
            if kind == 0:
                assert h.HcommLocalCopyOnThread(gpu_thread, dst, src, nbytes) == 0
            else:
                assert h.HcommLocalReduceOnThread(gpu_thread, dst, src, nbytes // 2, dt, oracle.SUM) == 0
        assert h.HcommBatchModeEnd(None) == 0
    h.HcommGfxThreadSynchronize(gpu_thread)
    log = h.launch_log(gpu_thread)
    assert len(log) == len(steps) == 15
    assert all(r.nseg == n for r in log)
    for r in range(n):
        assert_same(from_dev(d_out[r], host_in[r]), want_out[r], dt)
        assert_same(from_dev(d_in[r], host_in[r]), want_in[r], dt)


def test_plan_from_a_callers_op_list(gpu_thread):
    """HcommGfxPlanCreateFromOps: the oracle's own per-rank programs, handed over as an op list, replay to the oracle's
    result; so does a schedule written by hand here (a two-rank exchange through the communication buffers)."""
    for name, n, count, dtype in (("nhr_ar", 6, 70001, "fp32"), ("chunk_mesh", 4, 40009, "bf16"), ("nb_rs", 5, 9999, "int32")):
        dt = DT[dtype]
        say("op list", name, n, count, dtype)
        in_count, out_count = buffer_counts(name, n, count)
        host_in = [gen(dt, in_count, 7000 + r) for r in range(n)]
        want_in = [x.copy() for x in host_in]
        want_out = [np.zeros(out_count, host_in[0].dtype) for _ in range(n)]
        sb = h.scratch_bytes(ALGS[name][0], n, count, dt)
        want_scr = [np.zeros(sb, np.uint8) for _ in range(n)] if sb else None
        oracle.run(ALGS[name][1], want_in, want_out, count, dt, oracle.SUM, scratch=want_scr)
        d_in = [to_dev(x) for x in host_in]
        d_out = [to_dev(np.zeros(out_count, host_in[0].dtype)) for _ in range(n)]
        d_scr = [to_dev(np.zeros(sb, np.uint8)) for _ in range(n)] if sb else None
        bufs = {0: [t.data_ptr() for t in d_in], 1: [t.data_ptr() for t in d_out]}
        if sb:
            bufs[2] = [t.data_ptr() for t in d_scr]
        plan = h.OpListPlan(oracle.trace(ALGS[name][1], n, count, dt), n, bufs, dt, oracle.SUM)
        assert plan.run(gpu_thread) == 0
        assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
        for r in range(n):
            assert_same(from_dev(d_out[r], want_out[r]), want_out[r], dt, "%s out[%d]" % (name, r))
            assert_same(from_dev(d_in[r], host_in[r]), want_in[r], dt, "%s in[%d]" % (name, r))
        plan.destroy()
    # by hand: each of two ranks parks its input in the other's communication buffer, then folds it into its output
    count, dt = 50001, oracle.F32
    nb = count * 4
    a, b = gen(dt, count, 1), gen(dt, count, 2)
    ops = [(0, 0, 0, 1, 0, 0, 0, 0, nb), (0, 0, 1, 1, 0, 1, 0, 0, nb),          # out[r] = in[r]
           (0, 0, 0, 2, 0, 1, 0, 0, nb), (0, 0, 1, 2, 0, 0, 0, 0, nb),          # scratch[r] = in[peer]
           (1, 1, 0, 1, 0, 0, 2, 0, nb), (1, 1, 1, 1, 0, 1, 2, 0, nb)]          # out[r] += scratch[r]
    assert h.oplist_check(ops, 2, h.Expect.ALLREDUCE, count, 4)[:2] == (0, 0)
    d_in = [to_dev(a), to_dev(b)]
    d_out = [to_dev(np.zeros(count, np.float32)) for _ in range(2)]
    d_scr = [to_dev(np.zeros(count, np.float32)) for _ in range(2)]
    plan = h.OpListPlan(ops, 2, {0: [t.data_ptr() for t in d_in], 1: [t.data_ptr() for t in d_out],
                                 2: [t.data_ptr() for t in d_scr]}, dt, oracle.SUM)
    assert plan.info.launches == 2
    assert plan.run(gpu_thread) == 0
    assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
    assert_same(from_dev(d_out[0], a), a + b, dt, "out[0]")
    assert_same(from_dev(d_out[1], a), b + a, dt, "out[1]")
    plan.destroy()


def test_randomized_shapes(gpu_thread):
    """A fixed-seed sample of (algorithm, rank count, ragged element count, type, operation, lowering): every buffer
    bit-exact against the oracle.  Counts are drawn around the places where the kernels change path: the 16-byte
    vector, the 16 KiB tile, the 128-byte slice alignment, the small-message thresholds."""
    rng = np.random.default_rng(20240607)
    names = sorted(ALGS)
    interesting = [1, 2, 3, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 4095, 4096, 4097, 8191, 8192,
                   16383, 16385, 65535, 65537, 131071, 262145]
    done = 0
    while done < 250:
        name = names[rng.integers(len(names))]
        n = int(rng.integers(1, 17))
        if name in ("local_reduce", "doubling"):
            n = 1 << int(rng.integers(0, 5))
            if name == "local_reduce" and done % 5 == 0:
                n = 3
        base = interesting[rng.integers(len(interesting))]
        count = int(base * rng.integers(1, 4) + rng.integers(0, 3))
        dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
        op = ["sum", "max", "min", "prod"][rng.integers(4)]
        if op == "prod" and dtype in ("int16", "bf16"):        # the reference refuses these two (param_check.cc:327-343)
            continue
        lowering = h.Lowering.FUSED if (name in FUSABLE and rng.integers(2)) else h.Lowering.STEPWISE
        say("random", done, name, n, count, dtype, op, lowering)
        run_case(gpu_thread, name, lowering, n, count, dtype, op, seed=done)
        done += 1
