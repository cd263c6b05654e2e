"""The library loaded as a NIC plugin, the way the reference's plugin manager loads one (dlopen of the .so, dlsym of
HcommNicPluginGetInfo / CreateEndpoint / CreateChannel, nic_plugin_manager.cc:113-151), and its channel table called
the way the host adapter calls it (ch->GetNicOps()->writeReduceOnThread(ch->GetNicCtx(), thread, ...),
cpu_primitives_c_adpt.cc:320-340): results against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import oracle
import hcomm_amd as h
from hcomm_amd import nic_plugin as P
from util import DT, OPS, assert_same, from_dev, gen, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture()
def channel():
    code, ep_ctx, ep = P.create_endpoint(P.endpoint_desc())
    assert code == 0 and ep.init(ep_ctx) == 0
    code, ch_ctx, ch = P.create_channel(ep_ctx, P.channel_desc(2))
    assert code == 0 and ch.init(ch_ctx) == 0
    yield ch_ctx, ch
    assert ch.destroy(ch_ctx) == 0
    assert ep.destroy(ep_ctx) == 0


@pytest.mark.parametrize("dtype,op,count", [("bf16", "sum", 1 << 20), ("fp32", "max", 100003), ("int8", "min", 70001),
                                            ("fp16", "sum", 4099), ("int32", "sum", 1 << 18), ("fp32", "sum", 0)])
def test_write_and_read_reduce_through_the_channel_table(gpu_thread, channel, dtype, op, count):
    ch_ctx, ch = channel
    dt, o = DT[dtype], OPS[op]
    a, b = gen(dt, count + 8, 11, "special" if dtype in ("bf16", "fp32", "fp16") else "default"), gen(dt, count + 8, 142, "wide")
    want = a.copy()
    with np.errstate(all="ignore"):
        oracle.reduce(want[:count], b[:count].copy(), dt, o)
    for entry in (ch.writeReduceOnThread, ch.readReduceOnThread):
        d_a, d_b = to_dev(a), to_dev(b)
        assert entry(ch_ctx, gpu_thread, d_a.data_ptr(), d_b.data_ptr(), count, dt, o) == 0
        assert h.HcommGfxThreadSynchronize(gpu_thread) == 0
        assert_same(from_dev(d_a, a), want, dt, "%s %s" % (dtype, op), nan_bits=op in ("max", "min"))
        assert_same(from_dev(d_b, b), b, dt, "src untouched", nan_bits=True)


def test_copies_and_descriptor_batches_through_the_channel_table(gpu_thread, channel):
    ch_ctx, ch = channel
    dt = oracle.F32
    bufs = [gen(dt, 50001, 200 + i) for i in range(8)]
    dev = [to_dev(x) for x in bufs]
    nbytes = bufs[0].nbytes
    # dev[1] = dev[0] (write), dev[3] = dev[2] (read), both non-blocking twins on 4 and 5 / 6 and 7
    assert ch.writeOnThread(ch_ctx, gpu_thread, dev[1].data_ptr(), dev[0].data_ptr(), nbytes) == 0
    assert ch.readOnThread(ch_ctx, gpu_thread, dev[3].data_ptr(), dev[2].data_ptr(), nbytes) == 0
    assert ch.writeNbiOnThread(ch_ctx, gpu_thread, dev[5].data_ptr(), dev[4].data_ptr(), nbytes) == 0
    assert ch.readNbiOnThread(ch_ctx, gpu_thread, dev[7].data_ptr(), dev[6].data_ptr(), nbytes) == 0
    assert ch.drainOnThread(ch_ctx, gpu_thread) == 0
    h.HcommGfxThreadSynchronize(gpu_thread)
    for i in (0, 2, 4, 6):
        assert_same(from_dev(dev[i + 1], bufs[i]), bufs[i], dt, "copy %d" % i)
    # one descriptor batch: dev[1] += dev[2] and dev[3] = max(dev[3], dev[4]) become one launch each kind
    h.HcommGfxLaunchLogClear(gpu_thread)
    descs = (h.BatchTransferDesc * 3)(
        h.desc_reduce(dev[1].data_ptr(), dev[2].data_ptr(), 50001, dt, oracle.SUM),
        h.desc_reduce(dev[5].data_ptr(), dev[6].data_ptr(), 50001, dt, oracle.SUM, read=True),
        h.desc_copy(dev[7].data_ptr(), dev[0].data_ptr(), nbytes))
    assert ch.batchTransferOnThread(ch_ctx, gpu_thread, descs, 3) == 0
    h.HcommGfxThreadSynchronize(gpu_thread)
    assert [(r.kind, r.nseg) for r in h.launch_log(gpu_thread)] == [(h.Kernel.REDUCE2, 2), (h.Kernel.COPY, 1)]
    assert_same(from_dev(dev[1], bufs[0]), bufs[0] + bufs[2], dt, "batch reduce 0")
    assert_same(from_dev(dev[5], bufs[0]), bufs[4] + bufs[6], dt, "batch reduce 1")
    assert_same(from_dev(dev[7], bufs[0]), bufs[0], dt, "batch copy")


def test_channel_notifies_order_two_threads(gpu_thread, channel):
    """Thread A writes, records the channel's notify; thread B waits for it and reads what A wrote."""
    ch_ctx, ch = channel
    code, (tb,) = h.HcommThreadAlloc(h.CommEngine.CPU_TS, 1, 0)
    assert code == 0
    try:
        a = gen(oracle.F32, 1 << 22, 5)
        d_a, d_b, d_c = to_dev(a), to_dev(np.zeros_like(a)), to_dev(np.zeros_like(a))
        assert ch.notifyWaitOnThread(ch_ctx, tb, 0, 1) == h.HcclResult.E_TIMEOUT           # nothing recorded yet
        assert ch.writeOnThread(ch_ctx, gpu_thread, d_b.data_ptr(), d_a.data_ptr(), a.nbytes) == 0
        assert ch.notifyRecordOnThread(ch_ctx, gpu_thread, 0) == 0
        assert ch.notifyWaitOnThread(ch_ctx, tb, 0, 10) == 0
        assert ch.readOnThread(ch_ctx, tb, d_c.data_ptr(), d_b.data_ptr(), a.nbytes) == 0
        assert h.HcommGfxThreadSynchronize(tb) == 0
        assert_same(from_dev(d_c, a), a, oracle.F32, "read after notify")
        assert ch.notifyWaitOnThread(ch_ctx, tb, 0, 1) == h.HcclResult.E_TIMEOUT           # the record is consumed
    finally:
        h.HcommGfxThreadSynchronize(gpu_thread)
        h.HcommThreadFree([tb])
