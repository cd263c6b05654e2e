"""Step-wise plans lowered piece by piece (steps that write more than the memory-side cache keeps are run as all steps
on the first part of every slice, then all steps on the second, ...): with the size aimed at lowered from 128 MiB to a
few KiB, schedules of every kind at test sizes take that lowering where their operations are whole slices, and all 2N
buffers (and the communication buffers) still hold what the CPU oracle's replay leaves there, guard bytes included."""
import pytest

import hcomm_amd as h
from test_gpu_collectives import ALGS, run_case, say
from util import DT

pytestmark = pytest.mark.gpu

CASES = [
    # alg, n, count, dtype, op
    ("ring_ar", 8, 1000003, "bf16", "sum"),         # ragged last slice
    ("ring_ar", 5, 400009, "fp32", "max"),
    ("ring_ar", 3, 1 << 20, "int8", "sum"),
    ("ring_rs_stage", 7, 1000003, "fp32", "prod"),  # benchmark config 5a, scaled down
    ("ring_rs_stage", 7, 1000003, "int8", "sum"),
    ("mesh_oneshot", 8, 300007, "fp16", "sum"),
    ("mesh_ascending", 5, 300007, "bf16", "min"),
    ("mesh_rs", 7, 100003, "int32", "sum"),
    ("ring_rs", 8, 100003, "fp32", "sum"),
    ("chunk_mesh", 7, 300007, "fp32", "sum"),       # sub-chunks nest inside slices: stays as it is
    ("rhd_ar", 8, 400009, "int32", "sum"),          # nested ranges: stays as it is
    ("nhr_ar", 5, 400009, "bf16", "sum"),
    ("local_reduce", 8, 400009, "fp32", "sum"),
]


@pytest.mark.parametrize("aim", [4096, 65536])
@pytest.mark.parametrize("alg,n,count,dtype,op", CASES)
def test_plans_cut_into_pieces_leave_the_oracles_bytes(gpu_thread, alg, n, count, dtype, op, aim):
    say("pieces", alg, n, count, dtype, op, aim)
    whole = run_case(gpu_thread, alg, h.Lowering.STEPWISE, n, count, dtype, op, seed=21)
    before = h.HcommGfxSetPieceBytes(aim)
    try:
        cut = run_case(gpu_thread, alg, h.Lowering.STEPWISE, n, count, dtype, op, seed=21)
    finally:
        assert h.HcommGfxSetPieceBytes(before) == aim
    assert cut[1:] == whole[1:]                     # same algorithmic and moved bytes
    if alg in ("ring_ar", "ring_rs_stage"):   # slices on 128-byte boundaries: every two ranges the same or apart
        assert cut[0] > whole[0], "expected the piece-wise lowering for %s" % alg
    if alg in ("rhd_ar", "nhr_ar"):
        assert cut[0] == whole[0], "%s nests ranges and must keep one launch per step" % alg


@pytest.mark.parametrize("alg,n,count,dtype,op", [("ring_ar", 8, 1000003, "bf16", "sum"), ("ring_rs_stage", 7, 1000003, "int8", "sum"),
                                                  ("rhd_ar", 6, 100003, "fp32", "sum")])
def test_a_whole_collective_in_one_batch_is_cut_into_pieces_too(alg, n, count, dtype, op):
    """The same lowering behind the reference's boundary: a thread per rank, posts and waits, everything inside one
    HcommBatchModeStart / End pair - End's rounds are the steps it cuts."""
    from test_gpu_via_primitives import drive
    say("pieces, one batch over a thread per rank", alg, n, count, dtype, op)
    code, threads = h.HcommThreadAlloc(h.CommEngine.CPU_TS, n, 16)
    assert code == 0
    before = h.HcommGfxSetPieceBytes(8192)
    try:
        for t in threads:
            h.HcommGfxLaunchLogClear(t)
        drive("threads_batched", None, threads, alg, n, count, dtype, op)
        cut = len(h.launch_log(threads[0]))
        h.HcommGfxLaunchLogClear(threads[0])
        drive("one_batch", threads[0], None, alg, n, count, dtype, op)     # the same on one thread, without notifies
        cut_plain = len(h.launch_log(threads[0]))
        h.HcommGfxSetPieceBytes(0)
        h.HcommGfxLaunchLogClear(threads[0])
        drive("threads_batched", None, threads, alg, n, count, dtype, op)
        whole = len(h.launch_log(threads[0]))
        assert (cut > whole) == (alg != "rhd_ar")
        assert (cut_plain > whole) == (alg != "rhd_ar")
    finally:
        h.HcommGfxSetPieceBytes(before)
        for t in threads:
            h.HcommGfxThreadSynchronize(t)
        h.HcommThreadFree(threads)


def test_randomized_shapes_with_pieces_and_both_directions_forced(gpu_thread):
    """A fixed-seed sample of (algorithm, rank count, ragged element count, type, operation) step-wise, each with a
    random size from which steps are cut into pieces and from which launches walk against their producers - both
    far below any test size - against the oracle, all buffers, guard bytes included."""
    import numpy as np
    rng = np.random.default_rng(20250911)
    names = sorted(ALGS)
    interesting = [1, 7, 16, 33, 127, 129, 4095, 4097, 8192, 16385, 65537, 131071, 262145]
    before = h.HcommGfxSetAlternateBytes(1), h.HcommGfxSetPieceBytes(4096)
    try:
        done = 0
        while done < 120:
            name = names[rng.integers(len(names))]
            n = int(rng.integers(1, 17))
            if name in ("local_reduce", "doubling"):
                n = 1 << int(rng.integers(0, 5))
            count = int(interesting[rng.integers(len(interesting))] * rng.integers(1, 4) + rng.integers(0, 3))
            dtype = ["int8", "int16", "int32", "fp16", "fp32", "bf16"][rng.integers(6)]
            op = ["sum", "max", "min", "prod"][rng.integers(4)]
            if op == "prod" and dtype in ("int16", "bf16"):        # the reference refuses these two (param_check.cc:327-343)
                continue
            h.HcommGfxSetAlternateBytes([1, 4096, 65536][rng.integers(3)])
            h.HcommGfxSetPieceBytes([512, 4096, 65536][rng.integers(3)])
            say("random pieces", done, name, n, count, dtype, op)
            run_case(gpu_thread, name, h.Lowering.STEPWISE, n, count, dtype, op, seed=done)
            done += 1
    finally:
        h.HcommGfxSetAlternateBytes(before[0])
        h.HcommGfxSetPieceBytes(before[1])
