"""The benchmark configurations at their full sizes on the GPU, checked through what does not depend on
size: closed forms computed independently on the GPU by torch (exact integer sums / max / min, every rank's
output identical), and - for floating point - the CPU oracle run on the same inputs with all host cores."""
import sys

import numpy as np
import pytest

import oracle
import hcomm_amd as h

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_plan(thread, alg, lowering, ins, outs, count, dt, op):
    import torch
    torch.cuda.synchronize()
    plan = h.Plan(alg, lowering, [t.data_ptr() for t in ins], None if outs is None else [t.data_ptr() for t in outs],
                  count, dt, op)
    try:
        assert plan.run(thread) == 0
        assert h.HcommGfxThreadSynchronize(thread) == 0
        return plan.info
    finally:
        plan.destroy()


@pytest.mark.parametrize("lowering", [h.Lowering.STEPWISE, h.Lowering.FUSED])
@pytest.mark.parametrize("opname", ["sum", "max", "min"])
def test_config3_rhd_int32_16_ranks_128MiB(gpu_thread, opname, lowering):
    """RHD allreduce, int32, 16 ranks x 33,554,432 elements, values in [-2^20, 2^20]: bit-exact closed form."""
    import torch
    n, count = 16, 33554432
    say("cfg3", opname, lowering)
    g = torch.Generator(device="cuda")
    ins = []
    for r in range(n):
        g.manual_seed(300 + r)
        ins.append(torch.randint(-(1 << 20), (1 << 20) + 1, (count,), generator=g, device="cuda", dtype=torch.int32))
    if opname == "sum":
        want = torch.zeros(count, dtype=torch.int32, device="cuda")
        for x in ins:
            want += x           # |sum| <= 16 * 2^20 < 2^31: exact in any order
    else:
        want = ins[0].clone()
        for x in ins[1:]:
            want = torch.maximum(want, x) if opname == "max" else torch.minimum(want, x)
    outs = [torch.full((count,), -7, dtype=torch.int32, device="cuda") for _ in range(n)]
    op = {"sum": oracle.SUM, "max": oracle.MAX, "min": oracle.MIN}[opname]
    info = run_plan(gpu_thread, h.Alg.ALLREDUCE_RHD, lowering, ins, outs, count, oracle.I32, op)
    assert info.algorithmicBytes == 10334765056
    assert info.launches == (10 if lowering == h.Lowering.STEPWISE else 1)   # 9 steps; the last gather (1 GiB) in two launches
    for r in range(n):
        assert torch.equal(outs[r], want), "out[%d]" % r


@pytest.mark.parametrize("lowering", [h.Lowering.STEPWISE, h.Lowering.FUSED])
def test_config5b_ring_rs_int8_7_ranks_uneven(gpu_thread, lowering):
    """Ring reduce-scatter stage, int8 SUM, 7 ranks x 100,000,003 elements (last slice 14,285,059 bytes, odd):
    rank r's slice r equals the exact sum; all other bytes of every buffer equal what the oracle leaves there."""
    import torch
    n, count = 7, 100000003
    say("cfg5b", lowering)
    g = torch.Generator(device="cuda")
    pristine = []
    for r in range(n):
        g.manual_seed(500 + r)
        pristine.append(torch.randint(-8, 9, (count,), generator=g, device="cuda", dtype=torch.int8))
    ins = [x.clone() for x in pristine]
    info = run_plan(gpu_thread, h.Alg.REDUCE_SCATTER_RING, lowering, ins, None, count, oracle.I8, oracle.SUM)
    assert info.algorithmicBytes == 1800000054
    total = torch.zeros(count, dtype=torch.int8, device="cuda")
    for x in pristine:
        total += x               # |sum| <= 56: no wrap
    sl = oracle.slices_ring(count, 1, n)
    assert sl[6] == (85714944, 14285059)
    for r in range(n):
        lo, hi = sl[r][0], sl[r][0] + sl[r][1]
        assert torch.equal(ins[r][lo:hi], total[lo:hi]), "slice %d of rank %d" % (r, r)
    # every byte of every buffer, including the partial sums left behind, against the oracle
    host = [x.cpu().numpy() for x in pristine]
    oracle.lib().orc_set_threads(16)
    oracle.run(oracle.ALG_RS_RING_STAGE, host, [np.zeros(1, np.int8)] * n, count, oracle.I8, oracle.SUM)
    oracle.lib().orc_set_threads(1)
    for r in range(n):
        assert np.array_equal(ins[r].cpu().numpy(), host[r]), "in[%d]" % r


@pytest.mark.parametrize("lowering", [h.Lowering.STEPWISE, h.Lowering.FUSED])
def test_config5a_ring_rs_fp32_prod_7_ranks_uneven(gpu_thread, lowering):
    """Ring reduce-scatter stage, fp32 PROD, 7 ranks x 100,000,003 elements in [0.99, 1.01]: bit-exact against
    the oracle's reference-order product (tolerance stated by the task: <= 1 ulp; observed: 0)."""
    import torch
    n, count = 7, 100000003
    say("cfg5a", lowering)
    g = torch.Generator(device="cuda")
    pristine = []
    for r in range(n):
        g.manual_seed(700 + r)
        pristine.append(torch.rand(count, generator=g, device="cuda", dtype=torch.float32) * 0.02 + 0.99)
    ins = [x.clone() for x in pristine]
    info = run_plan(gpu_thread, h.Alg.REDUCE_SCATTER_RING, lowering, ins, None, count, oracle.F32, oracle.PROD)
    assert info.algorithmicBytes == 7200000216
    host = [x.cpu().numpy() for x in pristine]
    oracle.lib().orc_set_threads(16)
    oracle.run(oracle.ALG_RS_RING_STAGE, host, [np.zeros(1, np.float32)] * n, count, oracle.F32, oracle.PROD)
    oracle.lib().orc_set_threads(1)
    for r in range(n):
        got = ins[r].cpu().numpy()
        assert np.array_equal(got.view(np.uint32), host[r].view(np.uint32)), "in[%d]" % r
    # sanity against an order-free bound: the product of 7 values in [0.99, 1.01] lies in [0.932, 1.073]
    sl = oracle.slices_ring(count, 4, n)
    for r in range(n):
        lo, hi = sl[r][0] // 4, (sl[r][0] + sl[r][1]) // 4
        assert float(ins[r][lo:hi].min()) > 0.93 and float(ins[r][lo:hi].max()) < 1.08


@pytest.mark.parametrize("lowering", [h.Lowering.STEPWISE, h.Lowering.FUSED])
def test_config2_ring_bf16_8_ranks_128MiB(gpu_thread, lowering):
    """Ring allreduce SUM bf16, 8 ranks x 67,108,864 elements, N(0,1)*1e-3: all 16 buffers bit-exact against
    the oracle (task tolerance: <= 2 bf16 ulps; observed: 0), all outputs identical across ranks."""
    import torch
    n, count = 8, 67108864
    say("cfg2", lowering)
    g = torch.Generator(device="cuda")
    pristine = []
    for r in range(n):
        g.manual_seed(1234 + r)
        pristine.append((torch.randn(count, generator=g, device="cuda", dtype=torch.float32) * 1e-3)
                        .to(torch.bfloat16).view(torch.int16))
    ins = [x.clone() for x in pristine]
    outs = [torch.zeros(count, dtype=torch.int16, device="cuda") for _ in range(n)]
    info = run_plan(gpu_thread, h.Alg.ALLREDUCE_RING, lowering, ins, outs, count, oracle.BF16, oracle.SUM)
    assert info.algorithmicBytes == 4966055936
    for r in range(1, n):
        assert torch.equal(outs[r], outs[0])
    host_in = [x.cpu().numpy().view(np.uint16) for x in pristine]
    host_out = [np.zeros(count, np.uint16) for _ in range(n)]
    oracle.lib().orc_set_threads(16)
    oracle.run(oracle.ALG_ALLREDUCE_RING, host_in, host_out, count, oracle.BF16, oracle.SUM)
    oracle.lib().orc_set_threads(1)
    assert np.array_equal(outs[0].cpu().numpy().view(np.uint16), host_out[0])
    for r in range(n):
        assert np.array_equal(ins[r].cpu().numpy().view(np.uint16), host_in[r]), "in[%d]" % r
    # the bf16 result is within the accumulated rounding of an fp32 sum: 7 roundings of <= 2^-9 relative each
    f32 = sum(p.view(torch.bfloat16).float() for p in pristine)
    err = (outs[0].view(torch.bfloat16).float() - f32).abs().max().item()
    assert err < 7 * 2.0 ** -8 * 8e-3


def test_config4_mesh_oneshot_fp16_sweep(gpu_thread):
    """Mesh one-shot allreduce SUM fp16, 8 ranks, 4 KiB .. 4 MiB per rank: both lowerings bit-exact against the
    oracle at every size (each rank folds in its own order r, r+1, ..., so ranks may differ in the last ulp)."""
    from util import assert_same, from_dev, gen, to_dev
    n = 8
    for m in [1 << s for s in range(12, 23)]:
        count = m // 2
        host_in = [gen(oracle.F16, count, 40 + r) for r in range(n)]
        want_out = [np.zeros(count, np.uint16) for _ in range(n)]
        oracle.run(oracle.ALG_ALLREDUCE_MESH_ONESHOT, [x.copy() for x in host_in], want_out, count, oracle.F16, oracle.SUM)
        for lowering in (h.Lowering.STEPWISE, h.Lowering.FUSED):
            say("cfg4", m, lowering)
            d_in = [to_dev(x) for x in host_in]
            d_out = [to_dev(np.zeros(count, np.uint16)) for _ in range(n)]
            info = run_plan(gpu_thread, h.Alg.ALLREDUCE_MESH_ONESHOT, lowering, d_in, d_out, count, oracle.F16, oracle.SUM)
            assert info.launches == (8 if lowering == h.Lowering.STEPWISE else 1)
            if lowering == h.Lowering.FUSED:
                assert info.movedBytes == 72 * m
            for r in range(n):
                assert_same(from_dev(d_out[r], want_out[r]), want_out[r], oracle.F16, "m=%d out[%d]" % (m, r))
                assert_same(from_dev(d_in[r], host_in[r]), host_in[r], oracle.F16, "inputs untouched")


@pytest.mark.parametrize("lowering", [h.Lowering.STEPWISE, h.Lowering.FUSED])
@pytest.mark.parametrize("n,count", [(16, 33554432), (7, 25000003)])
@pytest.mark.parametrize("algname", ["nhr", "nb"])
def test_nhr_and_nb_int32_full_size_closed_form(gpu_thread, algname, n, count, lowering):
    """NHR / NB allreduce at benchmark size (16 x 128 MiB) and at a ragged non-power-of-two shape: exact int32
    sums computed independently by torch; every rank's output identical."""
    import torch
    say("full", algname, n, count, lowering)
    g = torch.Generator(device="cuda")
    ins = []
    want = torch.zeros(count, dtype=torch.int32, device="cuda")
    for r in range(n):
        g.manual_seed(700 + r)
        ins.append(torch.randint(-(1 << 20), (1 << 20) + 1, (count,), generator=g, device="cuda", dtype=torch.int32))
        want += ins[-1]
    outs = [torch.full((count,), -7, dtype=torch.int32, device="cuda") for _ in range(n)]
    alg = h.Alg.ALLREDUCE_NHR if algname == "nhr" else h.Alg.ALLREDUCE_NB
    info = run_plan(gpu_thread, alg, lowering, ins, outs, count, oracle.I32, oracle.SUM)
    steps = (n - 1).bit_length()
    if lowering == h.Lowering.FUSED:
        assert info.launches == 1
    elif algname == "nhr":      # touching slices are merged: one segment or two per rank, one launch per step (a copy
        assert 2 * steps + 1 <= info.launches <= 2 * steps + 3   # step that writes more than 512 MiB is cut)
    else:                       # NB keeps its slices apart: a step of 16 ranks x 8 slices needs 2 launches of 64 segments
        assert info.launches >= 2 * steps + 1
    for r in range(n):
        assert torch.equal(outs[r], want), "out[%d]" % r
    del ins, outs, want
    torch.cuda.empty_cache()


@pytest.mark.parametrize("algname,lowering", [
    ("local_reduce", h.Lowering.FUSED), ("chunk_mesh", h.Lowering.FUSED), ("local_reduce_rs", h.Lowering.FUSED),
    ("ring", h.Lowering.FUSED_KEEP_INPUTS), ("rhd", h.Lowering.FUSED_KEEP_INPUTS), ("nhr", h.Lowering.FUSED_KEEP_INPUTS),
    ("nb", h.Lowering.FUSED_KEEP_INPUTS), ("mesh_rs", h.Lowering.FUSED_KEEP_INPUTS),
])
def test_lowerings_that_only_read_the_inputs_full_size_closed_form(gpu_thread, algname, lowering):
    """128 MiB of int32 per rank on 8 ranks (reduce-scatters: 8 slices of 16 MiB): every output equals the exact
    sum, computed independently by torch, and every input is bit for bit what it was."""
    import torch
    n = 8
    scatter = algname in ("local_reduce_rs", "mesh_rs")
    count = (1 << 22) if scatter else (1 << 25)
    alg = {"local_reduce": h.Alg.ALLREDUCE_LOCAL_REDUCE, "chunk_mesh": h.Alg.ALLREDUCE_CHUNK_MESH,
           "local_reduce_rs": h.Alg.REDUCE_SCATTER_LOCAL_REDUCE, "ring": h.Alg.ALLREDUCE_RING, "rhd": h.Alg.ALLREDUCE_RHD,
           "nhr": h.Alg.ALLREDUCE_NHR, "nb": h.Alg.ALLREDUCE_NB, "mesh_rs": h.Alg.REDUCE_SCATTER_MESH}[algname]
    say("read-only lowering, full size", algname, lowering)
    g = torch.Generator(device="cuda")
    ins = []
    for r in range(n):
        g.manual_seed(900 + r)
        ins.append(torch.randint(-(1 << 20), (1 << 20) + 1, ((n if scatter else 1) * count,), generator=g, device="cuda",
                                 dtype=torch.int32))
    before = [x.clone() for x in ins]
    want = torch.zeros_like(ins[0])
    for x in ins:
        want += x
    outs = [torch.full((count,), -7, dtype=torch.int32, device="cuda") for _ in range(n)]
    info = run_plan(gpu_thread, alg, lowering, ins, outs, count, oracle.I32, oracle.SUM)
    assert info.movedBytes == ((n + 1) * n * count * 4 if scatter else 2 * n * count * 4)
    for r in range(n):
        assert torch.equal(ins[r], before[r]), "in[%d]" % r
        assert torch.equal(outs[r], want[r * count:(r + 1) * count] if scatter else want), "out[%d]" % r
