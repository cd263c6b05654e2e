"""HcommGfxAllReduceLocalReduceNoAlloc (the deterministic mesh allreduce on the library's own per-GPU array, for
callers that cannot allocate) against HcommGfxPlanCreateEx + HcommGfxPlanRun with caller-supplied communication
buffers: same inputs, outputs compared bit for bit, two calls in a row, the second with a smaller message, so that
whatever the first call left in the array is there when the second runs."""
import sys

import numpy as np
import pytest

import hcomm_amd as h
import oracle
from util import DT, OPS, gen, to_dev

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def both(thread, n, count, dtype, op, seed):
    """Outputs of the plan with supplied communication buffers and of the no-alloc call, as numpy byte arrays."""
    import torch
    dt, o = DT[dtype], OPS[op]
    unit = h.DTYPE_SIZE[dt]
    host_in = [gen(dt, count, seed * 100 + r, "prod" if op == "prod" else "default") for r in range(n)]
    d_in = [to_dev(x) for x in host_in]
    outs = []
    # existing entry point: communication buffers from the caller
    sb = h.scratch_bytes(h.Alg.ALLREDUCE_LOCAL_REDUCE, n, count, dt)
    d_scr = [torch.zeros(max(sb, 1), dtype=torch.uint8, device="cuda") for _ in range(n)]
    d_out = [torch.full((max(count * unit, 1),), 0xA5, dtype=torch.uint8, device="cuda") for _ in range(n)]
    torch.cuda.synchronize()
    plan = h.Plan(h.Alg.ALLREDUCE_LOCAL_REDUCE, h.Lowering.STEPWISE, [t.data_ptr() for t in d_in],
                  [t.data_ptr() for t in d_out], count, dt, o, 0, [t.data_ptr() for t in d_scr])
    h.check(plan.run(thread), "HcommGfxPlanRun")
    h.check(h.HcommGfxThreadSynchronize(thread), "sync")
    outs.append([t.cpu().numpy()[:count * unit].copy() for t in d_out])
    plan.destroy()
    # the new one: nothing but inputs and outputs
    d_out2 = [torch.full((max(count * unit, 1),), 0x5A, dtype=torch.uint8, device="cuda") for _ in range(n)]
    torch.cuda.synchronize()
    h.check(h.HcommGfxAllReduceLocalReduceNoAlloc(thread, [t.data_ptr() for t in d_in], [t.data_ptr() for t in d_out2],
                                                   count, dt, o), "HcommGfxAllReduceLocalReduceNoAlloc")
    h.check(h.HcommGfxThreadSynchronize(thread), "sync")
    outs.append([t.cpu().numpy()[:count * unit].copy() for t in d_out2])
    for r in range(n):  # the inputs are only read
        assert np.array_equal(d_in[r].cpu().numpy(), np.ascontiguousarray(host_in[r]).view(np.uint8)), ("input changed", r)
    # and the oracle, so that two equal wrong answers do not pass
    want_in = [x.copy() for x in host_in]
    want_out = [np.zeros(count, host_in[0].dtype) for _ in range(n)]
    want_scr = [np.zeros(sb, np.uint8) for _ in range(n)] if sb else None
    oracle.run(oracle.ALG_ALLREDUCE_LOCAL_REDUCE, want_in, want_out, count, dt, o, scratch=want_scr)
    outs.append([np.ascontiguousarray(w).view(np.uint8) for w in want_out])
    return outs


@pytest.fixture(scope="module")
def thread():
    code, threads = h.HcommThreadAlloc(h.CommEngine.CPU_TS, 1, 0)
    h.check(code, "HcommThreadAlloc")
    yield threads[0]
    h.HcommThreadFree(threads)


@pytest.mark.parametrize("n,dtype,op,counts", [
    (8, "bf16", "sum", (1048576 + 37, 4099)),     # 2 MiB per rank, then 8 KiB: the array still holds the first call's slots
    (4, "fp32", "sum", (500001, 1000)),
    (8, "int32", "max", (262147, 262147 // 3)),
    (2, "fp16", "prod", (70001, 3)),
    (8, "int8", "sum", (3 * 1048576 + 5, 129)),
])
def test_no_alloc_matches_plan(thread, n, dtype, op, counts):
    for i, count in enumerate(counts):
        say("no_alloc case", n, dtype, op, count)
        plan_out, noalloc_out, want = both(thread, n, count, dtype, op, seed=7 + i)
        for r in range(n):
            assert np.array_equal(noalloc_out[r], plan_out[r]), ("no-alloc vs plan", n, dtype, op, count, r)
            assert np.array_equal(plan_out[r], want[r]), ("plan vs oracle", n, dtype, op, count, r)


def test_no_alloc_limits(thread):
    import torch
    dt = DT["bf16"]
    bufs = [torch.zeros(1 << 20, dtype=torch.uint8, device="cuda") for _ in range(16)]
    ptrs = [t.data_ptr() for t in bufs]
    # a message whose communication buffers do not fit the library's array: refused, nothing launched
    too_big = (h.NOALLOC_SCRATCH_BYTES // 8) // 2 + 4096
    assert h.HcommGfxAllReduceLocalReduceNoAlloc(thread, ptrs[:8], ptrs[8:], too_big, dt, OPS["sum"]) == h.HcclResult.E_PARA
    # more ranks than the entry point takes
    assert h.HcommGfxAllReduceLocalReduceNoAlloc(thread, ptrs[:16], ptrs[:16], 16, dt, OPS["sum"]) == h.HcclResult.E_PARA
    # count 0: nothing to do
    assert h.HcommGfxAllReduceLocalReduceNoAlloc(thread, ptrs[:8], ptrs[8:], 0, dt, OPS["sum"]) == h.HcclResult.SUCCESS
    h.check(h.HcommGfxThreadSynchronize(thread), "sync")
