"""Signed zeros, infinities, NaNs and denormals through every lowering of every schedule.

MAX and MIN keep dst on a tie and on an unordered comparison (hccl_task_reduce_process.cc:36-40,50-54; the stub's
reduce_op called with src1 = src, llt_hccl_stub.cc:4089-4095,2374), so on +0 against -0 and on anything against a NaN
the operand ROLES decide the bits of the result: a single-launch lowering that folds in the schedule's order but with
the running value in the wrong role (all_reduce_mesh_oneshot.cc:94-119 keeps it in dst, the ring of
reduce_scatter_ring.cc:207-304 hands it over as src) leaves other bits than the step-wise replay.  The inputs of
util.gen_special make such comparisons meet at every position of a chain or a tree, every rank's NaNs carry that
rank's payload, and for MAX / MIN all 2N buffers are compared bit for bit, NaN payloads and signs included.  For SUM
and PROD (inf - inf, 0 * inf, overflow, denormal results) two NaNs compare equal whatever their payload: which
operand's payload an addition passes on is the adder's choice, x86's and gfx950's differ, and the reference pins
neither."""
import numpy as np
import pytest

import oracle
import hcomm_amd as h
from util import DT, OPS, UNIT, assert_same, gen, to_dev
from test_gpu_collectives import ALGS, FUSABLE, FUSABLE_NO_SCRATCH, buffer_counts, say

pytestmark = pytest.mark.gpu

# single-launch lowerings that work on the user buffers alone and only read the inputs
USER_BUFFER = {"local_reduce", "chunk_mesh", "local_reduce_rs", "window_rs"}
# their tree launches read block d of every input with 128-bit accesses
NEEDS_16_BYTE_BLOCKS = {"local_reduce_rs", "window_rs"}

# (ranks, elements): below and above the sizes at which a launch changes kernel (host-resolved addresses up to 8
# inputs in 8 segments, 4 KiB tiles up to 1 MiB per segment or 256 KiB when partials are stored, 16 KiB tiles
# beyond), rank counts with and without a power of two, element tails
SHAPES = {
    "ring_ar": [(2, 4099), (5, 20011), (8, 70001), (3, 400003), (12, 4099)],
    "ring_rs_stage": [(3, 4099), (7, 50001), (3, 400003)],
    "rhd_ar": [(4, 4099), (6, 20011), (7, 70001), (3, 4099), (8, 20011), (12, 4099)],
    "mesh_oneshot": [(2, 4099), (5, 20011), (8, 4099), (3, 600007), (12, 4099)],
    "mesh_ascending": [(3, 4099), (8, 20011), (3, 600007)],
    "mesh_rs": [(4, 4099), (7, 5001)],
    "ring_rs": [(3, 4099), (8, 5001)],
    "local_reduce": [(2, 4099), (3, 20011), (8, 70001), (32, 160000)],
    "chunk_mesh": [(3, 4099), (8, 70001), (5, 600007)],
    "nhr_ar": [(3, 4099), (5, 20011), (8, 70001), (12, 4099)],
    "nhr_rs": [(5, 4099), (8, 5001)],
    "nb_ar": [(3, 4099), (6, 20011), (8, 70001), (12, 4099)],
    "nb_rs": [(5, 4099), (8, 5001)],
    "local_reduce_rs": [(3, 4104), (7, 5000), (8, 40000), (12, 4104)],
    "doubling": [(2, 4099), (8, 20011), (16, 4099)],
    "nhr_oneshot": [(3, 4099), (6, 20011), (8, 4099), (13, 4099), (5, 600007)],
    "window_rs": [(3, 4104), (7, 5000), (8, 40000), (12, 4104)],
}


def lowerings_of(alg, count, dtype):
    """The lowerings a schedule has for this shape: step-wise always; the single launch that reproduces the replay's
    writes into the inputs; the single launch that keeps them."""
    out = [h.Lowering.STEPWISE]
    fits = alg not in NEEDS_16_BYTE_BLOCKS or (count * UNIT[DT[dtype]]) % 16 == 0
    if (alg in FUSABLE or alg in FUSABLE_NO_SCRATCH or alg in USER_BUFFER) and fits:
        out.append(h.Lowering.FUSED)
    if (alg in FUSABLE or alg in USER_BUFFER or alg == "doubling") and alg != "ring_rs_stage" and fits:
        out.append(h.Lowering.FUSED_KEEP_INPUTS)
    return out


def run_special(thread, alg, lowering, n, count, dtype, op, seed):
    dt, o = DT[dtype], OPS[op]
    in_count, out_count = buffer_counts(alg, n, count)
    host_in = [gen(dt, in_count, seed + 131 * r, "special") for r in range(n)]
    sentinel = gen(dt, out_count, 999, "wide")
    want_in = [x.copy() for x in host_in]
    want_out = [sentinel.copy() for _ in range(n)]
    sb = h.scratch_bytes(ALGS[alg][0], n, count, dt)
    with np.errstate(all="ignore"):
        oracle.run(ALGS[alg][1], want_in, want_out, count, dt, o,
                   scratch=[np.zeros(sb, np.uint8) for _ in range(n)] if sb else None)
    inputs_kept = lowering == h.Lowering.FUSED_KEEP_INPUTS or (lowering == h.Lowering.FUSED and alg in USER_BUFFER)
    if inputs_kept:
        want_in = host_in
    d_in = [to_dev(x) for x in host_in]
    d_out = [to_dev(sentinel) for _ in range(n)]
    d_scr = [to_dev(np.zeros(sb, np.uint8)) for _ in range(n)] if sb and lowering == h.Lowering.STEPWISE else None
    plan = h.Plan(ALGS[alg][0], lowering, [t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out], count, dt, o, 0,
                  [t.data_ptr() for t in d_scr] if d_scr else None)
    try:
        if lowering != h.Lowering.STEPWISE and n > 1:
            assert all(r.kind in (h.Kernel.CHAIN, h.Kernel.TREE) for r in plan.launches()), "not a fold launch"
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        strict = op in ("max", "min")
        what = "%s n=%d count=%d %s %s lowering %d" % (alg, n, count, dtype, op, int(lowering))
        for r in range(n):
            got_in = d_in[r].cpu().numpy().view(host_in[r].dtype)
            got_out = d_out[r].cpu().numpy().view(sentinel.dtype)
            assert_same(got_in, want_in[r], dt, "%s in[%d]" % (what, r), nan_bits=strict)
            assert_same(got_out, want_out[r], dt, "%s out[%d]" % (what, r), nan_bits=strict)
    finally:
        plan.destroy()


@pytest.mark.parametrize("op", ["max", "min", "sum", "prod"])
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("alg", sorted(SHAPES))
def test_special_values_through_every_lowering(gpu_thread, alg, dtype, op):
    if op == "prod" and dtype == "bf16":
        pytest.skip("the reference's collectives refuse PROD on bf16 (param_check.cc:327-343) and so do the plans")
    for i, (n, count) in enumerate(SHAPES[alg]):
        for lowering in lowerings_of(alg, count, dtype):
            say("special", alg, n, count, dtype, op, "lowering", int(lowering))
            run_special(gpu_thread, alg, lowering, n, count, dtype, op, seed=1000 * i + 17)


@pytest.mark.parametrize("op", ["max", "min"])
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_special_values_through_the_k_way_reduce(gpu_thread, dtype, op):
    """HcommGfxReduceKOnThread (out = ((x0 (op) x1) (op) x2) ..., the running value in the dst role) with 2 .. 9
    inputs, small and large enough for each of the chain kernels."""
    dt, o = DT[dtype], OPS[op]
    for k, count in ((2, 4099), (3, 20011), (8, 4099), (9, 70001), (5, 1200007)):
        say("special reduce_k", k, count, dtype, op)
        srcs = [gen(dt, count, 40 + 131 * j, "special") for j in range(k)]
        want = srcs[0].copy()
        for j in range(1, k):
            oracle.reduce(want, srcs[j].copy(), dt, o)
        d_src = [to_dev(x) for x in srcs]
        d_out = to_dev(gen(dt, count, 999, "wide"))
        assert h.HcommGfxReduceKOnThread(gpu_thread, d_out.data_ptr(), [t.data_ptr() for t in d_src], count, dt, o) == 0
        assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
        assert_same(d_out.cpu().numpy().view(want.dtype), want, dt, "reduce_k k=%d" % k, nan_bits=True)
        for j in range(k):
            assert_same(d_src[j].cpu().numpy().view(want.dtype), srcs[j], dt, "src %d" % j, nan_bits=True)
