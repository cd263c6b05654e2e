"""ctypes binding of include/hcomm_gfx.h.

Every function here is a one-line call into libhcomm_gfx.so; there is no Python or CPU implementation of
any operation.  If the library is missing, importing this module raises - it never falls back.
"""
import ctypes as C
import os

try:
    # A process can hold only one HIP runtime.  PyTorch-ROCm ships its own libamdhip64 (same soname as the one
    # under /opt/rocm), and the dynamic loader shares it with this library only when torch was loaded first.
    import torch  # noqa: F401
except ImportError:  # a pure C / ctypes caller without torch uses the system runtime
    pass

__all__ = [
    "lib", "LIB_PATH", "plan_tree", "OpListKeepInputsPlan", "HcclResult", "HcommReduceOp", "HcommDataType", "CommEngine", "Alg", "Lowering", "Kernel",
    "LaunchRecord", "PlanInfo", "SchedOp", "Slice", "HcommError", "check",
    "HcommLocalCopyOnThread", "HcommLocalReduceOnThread", "HcommThreadAlloc", "HcommThreadFree",
    "HcommThreadAllocWithStream", "HcommThreadFreeWithStream", "HcommThreadNotifyRecordOnThread",
    "HcommThreadNotifyWaitOnThread", "HcommMemAlloc", "HcommMemFree", "HcommBatchModeStart", "HcommBatchModeEnd",
    "HcommGfxThreadSynchronize", "HcommGfxReduceKOnThread", "HcommGfxRecorderThreadAlloc", "launch_log",
    "HcommGfxLaunchLogClear", "calc_slices", "HcommGfxDataTypeSize", "Plan", "schedule_emit", "HcommGfxVersion", "HcommGfxSetDirectLaunches", "HcommGfxSetAlternateBytes", "HcommGfxSetPieceBytes",
    "DTYPE_SIZE", "HcommWriteOnThread", "HcommReadOnThread", "HcommWriteReduceOnThread", "HcommReadReduceOnThread",
    "HcommBatchTransferOnThread", "BatchTransferDesc", "TransferType", "desc_copy", "desc_reduce",
    "CheckReport", "Expect", "oplist_check", "schedule_check", "scratch_bytes",
    "HcommWriteNbiOnThread", "HcommReadNbiOnThread", "HcommSetNotifyWaitTimeOut",
    "HcommThreadNotifyWaitOnThreadWithDefaultTimeout", "HcommThreadResAcquireTimeOut", "HcommFenceOnThread",
    "HcommChannelFenceOnThread", "HcommChannelDrainOnThread",
    "HierPlan", "hier_emit", "hier_check", "DoubleRingPlan", "dbring_emit", "dbring_check",
    "OrderPreservedPlan", "order_preserved_emit", "order_preserved_check",
    "OrderPreservedSmallPlan", "order_preserved_small_emit", "order_preserved_small_check",
    "OrderPreservedAllReducePlan", "order_preserved_ar_emit", "order_preserved_ar_check", "OrderPreservedFusedPlan",
    "OrderPreservedHierAllReducePlan", "order_preserved_hier_ar_emit", "order_preserved_hier_ar_check",
    "OrderPreservedHierReduceScatterPlan", "order_preserved_hier_rs_emit", "order_preserved_hier_rs_check",
    "HierReduceScatterPlan", "hier_rs_emit", "hier_rs_check",
    "DoubleRingReduceScatterPlan", "dbring_rs_emit", "dbring_rs_check",
    "DoubleRingHierReduceScatterPlan", "dbring_hier_rs_emit", "dbring_hier_rs_check",
    "HcommGfxAllReduceLocalReduceNoAlloc", "NOALLOC_SCRATCH_BYTES", "NOALLOC_MAX_RANKS",
    "OpBasePlan", "OpListPlan", "opbase_emit", "opbase_check", "opbase_max_count", "BUF_USER_IN", "BUF_USER_OUT",
]

# HCOMM_GFX_LIB names another build of the library to bind (a debug build, a build with other compile-time settings)
LIB_PATH = os.environ.get("HCOMM_GFX_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc",
                                                            "libhcomm_gfx.so")
if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libhcomm_gfx.so is not built (%s); run `python -c 'import __graft_entry__ as g; g.build()'` or "
        "`make -C hcomm_amd/csrc`" % LIB_PATH)
lib = C.CDLL(LIB_PATH)


class HcclResult:
    SUCCESS, E_PARA, E_PTR, E_MEMORY, E_INTERNAL, E_NOT_SUPPORT, E_NOT_FOUND, E_UNAVAIL = range(8)
    E_TIMEOUT = 9
    E_RUNTIME = 15


class HcommReduceOp:
    SUM, PROD, MAX, MIN = 0, 1, 2, 3
    RESERVED = 255


class HcommDataType:
    INT8, INT16, INT32, FP16, FP32, INT64, UINT64, UINT8, UINT16, UINT32, FP64, BFP16, INT128 = range(13)
    HIF8, FP8E4M3, FP8E5M2, FP8E8M0 = 14, 15, 16, 17
    RESERVED = 255


DTYPE_SIZE = {HcommDataType.INT8: 1, HcommDataType.INT16: 2, HcommDataType.INT32: 4, HcommDataType.FP16: 2,
              HcommDataType.FP32: 4, HcommDataType.BFP16: 2}


class CommEngine:
    RESERVED, CPU, CPU_TS, AICPU, AICPU_TS, AIV, CCU = -1, 0, 1, 2, 3, 4, 5


class Alg:
    ALLREDUCE_RING, REDUCE_SCATTER_RING, ALLREDUCE_RHD, ALLREDUCE_MESH_ONESHOT, REDUCE_SCATTER_MESH, \
        REDUCE_SCATTER_RING_STANDALONE, ALLREDUCE_MESH_ONESHOT_ASCENDING, ALLREDUCE_LOCAL_REDUCE, \
        ALLREDUCE_CHUNK_MESH, ALLREDUCE_NHR, REDUCE_SCATTER_NHR, ALLREDUCE_NB, REDUCE_SCATTER_NB, \
        REDUCE_SCATTER_LOCAL_REDUCE, ALLREDUCE_DOUBLING, ALLREDUCE_NHR_ONESHOT, REDUCE_SCATTER_RHD, \
        REDUCE_SCATTER_WINDOW_HALVING = range(18)


class Lowering:
    STEPWISE, FUSED, FUSED_KEEP_INPUTS = 0, 1, 2


class Kernel:
    COPY, REDUCE2, CHAIN, TREE, BYTEWISE = range(5)


class LaunchRecord(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("dtype", C.c_uint32), ("op", C.c_uint32), ("nseg", C.c_uint32),
                ("bytes", C.c_uint64), ("blocks", C.c_uint64), ("rows", C.c_uint32), ("streaming", C.c_uint32),
                ("backwards", C.c_uint32), ("reserved", C.c_uint32)]


class PlanInfo(C.Structure):
    _fields_ = [("launches", C.c_uint32), ("steps", C.c_uint32), ("algorithmicBytes", C.c_uint64),
                ("movedBytes", C.c_uint64)]


class SchedOp(C.Structure):
    _fields_ = [("step", C.c_uint32), ("kind", C.c_uint32), ("rank", C.c_uint32), ("dstBuf", C.c_uint32),
                ("srcRank", C.c_uint32), ("srcBuf", C.c_uint32), ("dstOff", C.c_uint64), ("srcOff", C.c_uint64),
                ("bytes", C.c_uint64)]

    def astuple(self):
        return (self.step, self.kind, self.rank, self.dstBuf, self.dstOff, self.srcRank, self.srcBuf, self.srcOff,
                self.bytes)


class _DescRW(C.Structure):
    _fields_ = [("len", C.c_uint64), ("dst", C.c_void_p), ("src", C.c_void_p)]


class _DescReduce(C.Structure):
    _fields_ = [("count", C.c_uint64), ("dst", C.c_void_p), ("src", C.c_void_p), ("reduceOp", C.c_int),
                ("dataType", C.c_int)]


class _DescInfo(C.Union):
    _fields_ = [("raws", C.c_uint8 * 56), ("write", _DescRW), ("read", _DescRW), ("reduce", _DescReduce)]


class BatchTransferDesc(C.Structure):
    """HcommBatchTransferDesc (64 bytes)."""
    _fields_ = [("transType", C.c_int), ("reserved", C.c_uint8 * 4), ("transferInfo", _DescInfo)]


class TransferType:
    INVALID, WRITE, WRITE_REDUCE, WRITE_WITH_NOTIFY, WRITE_REDUCE_WITH_NOTIFY, READ, READ_REDUCE, NOTIFY_RECORD = \
        -1, 0, 1, 2, 3, 4, 5, 6


class Slice(C.Structure):
    _fields_ = [("offset", C.c_uint64), ("size", C.c_uint64)]


class HcommError(RuntimeError):
    def __init__(self, code, what):
        super().__init__("%s failed with HcclResult %d" % (what, code))
        self.code = code


def check(code, what="call"):
    if code != 0:
        raise HcommError(code, what)
    return code


def _sig(name, restype, *argtypes):
    f = getattr(lib, name)
    f.restype = restype
    f.argtypes = list(argtypes)
    return f


_u64, _u32, _i32, _vp = C.c_uint64, C.c_uint32, C.c_int32, C.c_void_p

HcommLocalCopyOnThread = _sig("HcommLocalCopyOnThread", _i32, _u64, _vp, _vp, _u64)
HcommLocalReduceOnThread = _sig("HcommLocalReduceOnThread", _i32, _u64, _vp, _vp, _u64, C.c_int, C.c_int)
_thread_alloc = _sig("HcommThreadAlloc", _i32, C.c_int, _u32, C.POINTER(_u32), C.POINTER(_u64))
_thread_free = _sig("HcommThreadFree", _i32, C.POINTER(_u64), _u32)
_thread_alloc_stream = _sig("HcommThreadAllocWithStream", _i32, C.c_int, _vp, _u32, C.POINTER(_u64))
_thread_free_stream = _sig("HcommThreadFreeWithStream", _i32, C.POINTER(_u64), _u32)
HcommThreadNotifyRecordOnThread = _sig("HcommThreadNotifyRecordOnThread", _i32, _u64, _u64, _u32)
HcommThreadNotifyWaitOnThread = _sig("HcommThreadNotifyWaitOnThread", _i32, _u64, _u32, _u32)
_mem_alloc = _sig("HcommMemAlloc", _i32, C.POINTER(_vp), C.c_size_t)
HcommMemFree = _sig("HcommMemFree", _i32, _vp)
HcommBatchModeStart = _sig("HcommBatchModeStart", _i32, C.c_char_p)
HcommBatchModeEnd = _sig("HcommBatchModeEnd", _i32, C.c_char_p)
HcommGfxThreadSynchronize = _sig("HcommGfxThreadSynchronize", _i32, _u64)
_reduce_k = _sig("HcommGfxReduceKOnThread", _i32, _u64, _vp, C.POINTER(_vp), _u32, _u64, C.c_int, C.c_int)
_recorder_alloc = _sig("HcommGfxRecorderThreadAlloc", _i32, C.POINTER(_u64))
_log_read = _sig("HcommGfxLaunchLogRead", _i32, _u64, C.POINTER(LaunchRecord), _u32, C.POINTER(_u32))
HcommGfxLaunchLogClear = _sig("HcommGfxLaunchLogClear", _i32, _u64)
_calc_slices = _sig("HcommGfxCalcSlices", _i32, _u64, _u32, _u32, C.POINTER(Slice))
HcommGfxDataTypeSize = _sig("HcommGfxDataTypeSize", _u32, C.c_int)
_plan_create = _sig("HcommGfxPlanCreateEx", _i32, C.c_int, C.c_int, _u32, C.POINTER(_vp), C.POINTER(_vp),
                    C.POINTER(_vp), _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))
_scratch_bytes = _sig("HcommGfxScratchBytes", _i32, C.c_int, _u32, _u64, C.c_int, C.POINTER(_u64))


_noalloc = _sig("HcommGfxAllReduceLocalReduceNoAlloc", _i32, _u64, _u32, C.POINTER(_vp), C.POINTER(_vp), _u64, C.c_int,
                C.c_int)
NOALLOC_SCRATCH_BYTES = 64 << 20
NOALLOC_MAX_RANKS = 8


def HcommGfxAllReduceLocalReduceNoAlloc(thread, in_ptrs, out_ptrs, count, dtype, op):
    """The deterministic mesh allreduce in one call, on the library's own communication buffers; returns the code."""
    n = len(in_ptrs)
    return _noalloc(thread, n, (_vp * n)(*in_ptrs), (_vp * n)(*out_ptrs), count, dtype, op)


def scratch_bytes(alg, n_ranks, count, dtype):
    b = _u64(0)
    check(_scratch_bytes(alg, n_ranks, count, dtype, C.byref(b)), "HcommGfxScratchBytes")
    return b.value
_plan_run = _sig("HcommGfxPlanRun", _i32, _vp, _u64)
_plan_run_range = _sig("HcommGfxPlanRunRange", _i32, _vp, _u64, _u32, _u32)
_plan_destroy = _sig("HcommGfxPlanDestroy", _i32, _vp)
_plan_graph = _sig("HcommGfxPlanSetGraphReplay", _i32, _vp, _i32)
_plan_info = _sig("HcommGfxPlanGetInfo", _i32, _vp, C.POINTER(PlanInfo))
_plan_launch = _sig("HcommGfxPlanGetLaunch", _i32, _vp, _u32, C.POINTER(LaunchRecord))
_plan_tree_segment = _sig("HcommGfxPlanGetTreeSegment", _i32, _vp, _u32, _u32, C.POINTER(_vp), _u32, C.POINTER(_u32),
                         C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_i32))
_sched_emit = _sig("HcommGfxScheduleEmitStrided", _i32, C.c_int, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp), _u64,
                   C.POINTER(_u64))
HcommWriteOnThread = _sig("HcommWriteOnThread", _i32, _u64, _u64, _vp, _vp, _u64)
HcommReadOnThread = _sig("HcommReadOnThread", _i32, _u64, _u64, _vp, _vp, _u64)
HcommWriteReduceOnThread = _sig("HcommWriteReduceOnThread", _i32, _u64, _u64, _vp, _vp, _u64, C.c_int, C.c_int)
HcommReadReduceOnThread = _sig("HcommReadReduceOnThread", _i32, _u64, _u64, _vp, _vp, _u64, C.c_int, C.c_int)
HcommWriteNbiOnThread = _sig("HcommWriteNbiOnThread", _i32, _u64, _u64, _vp, _vp, _u64)
HcommReadNbiOnThread = _sig("HcommReadNbiOnThread", _i32, _u64, _u64, _vp, _vp, _u64)
HcommSetNotifyWaitTimeOut = _sig("HcommSetNotifyWaitTimeOut", _i32, C.c_float)
HcommThreadNotifyWaitOnThreadWithDefaultTimeout = _sig("HcommThreadNotifyWaitOnThreadWithDefaultTimeout", _i32, _u64, _u32)
HcommThreadResAcquireTimeOut = _sig("HcommThreadResAcquireTimeOut", _i32, C.c_float)
HcommFenceOnThread = _sig("HcommFenceOnThread", _i32, _u64)
HcommChannelFenceOnThread = _sig("HcommChannelFenceOnThread", _i32, _u64, _u64)
HcommChannelDrainOnThread = _sig("HcommChannelDrainOnThread", _i32, _u64, _u64)
_batch_transfer = _sig("HcommBatchTransferOnThread", _i32, _u64, _u64, C.POINTER(BatchTransferDesc), _u32)
class CheckReport(C.Structure):
    _fields_ = [("conflicts", C.c_uint32), ("semanticErrors", C.c_uint32), ("message", C.c_char * 248)]


class Expect:
    ALLREDUCE, REDUCE_SCATTER_IN_PLACE, REDUCE_SCATTER_OUT, ALLREDUCE_USER, REDUCE_SCATTER_USER = 0, 1, 2, 3, 4


_oplist_check = _sig("HcommGfxOpListCheck", _i32, C.POINTER(SchedOp), _u64, _u32, C.c_int, _u64, _u64, _u32,
                     C.POINTER(CheckReport))
_sched_check = _sig("HcommGfxScheduleCheck", _i32, C.c_int, _u32, _u64, _u64, C.c_int, C.POINTER(CheckReport))


def oplist_check(ops, n_ranks, expect, count, unit, stride=0):
    """ops: tuples as returned by schedule_emit.  Returns (conflicts, semantic_errors, message)."""
    arr = (SchedOp * max(len(ops), 1))()
    for i, (step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes) in enumerate(ops):
        arr[i] = SchedOp(step, kind, rank, dbuf, srank, sbuf, doff, soff, nbytes)
    rep = CheckReport()
    check(_oplist_check(arr, len(ops), n_ranks, expect, count, stride, unit, C.byref(rep)), "HcommGfxOpListCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


def schedule_check(alg, n_ranks, count, dtype, stride=0):
    rep = CheckReport()
    check(_sched_check(alg, n_ranks, count, stride, dtype, C.byref(rep)), "HcommGfxScheduleCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


_version = _sig("HcommGfxVersion", C.c_char_p)


def HcommBatchTransferOnThread(thread, channel, descs):
    arr = (BatchTransferDesc * max(len(descs), 1))(*descs)
    return _batch_transfer(thread, channel, arr if descs else None, len(descs))


def desc_copy(dst, src, nbytes, read=False):
    d = BatchTransferDesc()
    d.transType = TransferType.READ if read else TransferType.WRITE
    d.transferInfo.write.len, d.transferInfo.write.dst, d.transferInfo.write.src = nbytes, dst, src
    return d


def desc_reduce(dst, src, count, dtype, op, read=False):
    d = BatchTransferDesc()
    d.transType = TransferType.READ_REDUCE if read else TransferType.WRITE_REDUCE
    r = d.transferInfo.reduce
    r.count, r.dst, r.src, r.reduceOp, r.dataType = count, dst, src, op, dtype
    return d


_set_direct = _sig("HcommGfxSetDirectLaunches", C.c_int32, C.c_int32)


def HcommGfxSetDirectLaunches(enable):
    """0: launches shaped from now on stay on the kernels large launches use; 1: the default.  Returns the previous setting."""
    return int(_set_direct(1 if enable else 0))


_set_alternate = _sig("HcommGfxSetAlternateBytes", C.c_uint64, C.c_uint64)


def HcommGfxSetAlternateBytes(nbytes):
    """Launches that write more than nbytes may walk their table backwards (0 = never); returns the previous value."""
    return _set_alternate(nbytes)


_set_piece = _sig("HcommGfxSetPieceBytes", C.c_uint64, C.c_uint64)


def HcommGfxSetPieceBytes(nbytes):
    """Step-wise plans created from now on cut steps that write more than 2 x nbytes into pieces of about nbytes
    (0 = never); returns the previous value."""
    return _set_piece(nbytes)


def HcommGfxVersion():
    return _version().decode()


def HcommThreadAlloc(engine=CommEngine.CPU_TS, thread_num=1, notify_num=0):
    """Returns (code, [handles])."""
    handles = (_u64 * max(thread_num, 1))()
    notif = (_u32 * 1)(notify_num)
    code = _thread_alloc(engine, thread_num, notif, handles)
    return code, list(handles)[:thread_num]


def HcommThreadFree(handles):
    arr = (_u64 * max(len(handles), 1))(*handles)
    return _thread_free(arr, len(handles))


def HcommThreadAllocWithStream(stream_ptr, notify_num=0, engine=CommEngine.CPU_TS):
    """stream_ptr: integer value of a hipStream_t (0 = default stream).  Returns (code, handle)."""
    h = _u64(0)
    code = _thread_alloc_stream(engine, _vp(stream_ptr), notify_num, C.byref(h))
    return code, h.value


def HcommThreadFreeWithStream(handles):
    arr = (_u64 * max(len(handles), 1))(*handles)
    return _thread_free_stream(arr, len(handles))


def HcommMemAlloc(size):
    p = _vp(0)
    code = _mem_alloc(C.byref(p), size)
    return code, (p.value or 0)


def HcommGfxReduceKOnThread(thread, dst, srcs, count, dtype, op):
    arr = (_vp * max(len(srcs), 1))(*srcs)
    return _reduce_k(thread, dst, arr, len(srcs), count, dtype, op)


def HcommGfxRecorderThreadAlloc():
    h = _u64(0)
    code = _recorder_alloc(C.byref(h))
    return code, h.value


def launch_log(thread):
    n = _u32(0)
    check(_log_read(thread, None, 0, C.byref(n)), "HcommGfxLaunchLogRead")
    recs = (LaunchRecord * max(n.value, 1))()
    check(_log_read(thread, recs, n.value, C.byref(n)), "HcommGfxLaunchLogRead")
    return [recs[i] for i in range(n.value)]


def calc_slices(count, unit, n):
    sl = (Slice * n)()
    check(_calc_slices(count, unit, n, sl), "HcommGfxCalcSlices")
    return [(s.offset, s.size) for s in sl]


def schedule_emit(alg, n_ranks, count, dtype, stride=0):
    n = _u64(0)
    check(_sched_emit(alg, n_ranks, count, stride, dtype, None, 0, C.byref(n)), "HcommGfxScheduleEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_sched_emit(alg, n_ranks, count, stride, dtype, ops, n.value, C.byref(n)), "HcommGfxScheduleEmit")
    return [ops[i].astuple() for i in range(n.value)]


class Plan:
    """HcommGfxPlan: build once, run many."""

    def __init__(self, alg, lowering, in_ptrs, out_ptrs, count, dtype, op, stride=0, scratch_ptrs=None):
        n = len(in_ptrs)
        self._in = (_vp * n)(*in_ptrs)
        self._out = (_vp * n)(*out_ptrs) if out_ptrs is not None else None
        self._scratch = (_vp * n)(*scratch_ptrs) if scratch_ptrs is not None else None
        p = _vp(0)
        check(_plan_create(alg, lowering, n, self._in, self._out, self._scratch, count, stride, dtype, op, C.byref(p)),
              "HcommGfxPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info

    def run(self, thread):
        return _plan_run(self._p, thread)

    def set_graph_replay(self, enable):
        return _plan_graph(self._p, 1 if enable else 0)

    def run_range(self, thread, first, n):
        return _plan_run_range(self._p, thread, first, n)

    def launches(self):
        out = []
        for i in range(self.info.launches):
            r = LaunchRecord()
            check(_plan_launch(self._p, i, C.byref(r)), "HcommGfxPlanGetLaunch")
            out.append(r)
        return out

    def destroy(self):
        if self._p is not None:
            _plan_destroy(self._p)
            self._p = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def plan_tree(plan, launch, segment, rank_of=None, with_owner=False):
    """(tree, offset, bytes) of one segment of a tree launch of any plan object: the nested [dst, src] lists the
    kernel's fold pattern makes of the leaf positions (level l folds position q + 2^l onto q, holes skipped); a leaf
    is the input pointer read there, or rank_of[pointer] when a mapping is given."""
    k, off, nbytes, owner = _u32(0), _u64(0), _u64(0), _i32(0)
    check(_plan_tree_segment(plan._p, launch, segment, None, 0, C.byref(k), C.byref(off), C.byref(nbytes),
                             C.byref(owner)), "HcommGfxPlanGetTreeSegment")
    leaves = (_vp * k.value)()
    check(_plan_tree_segment(plan._p, launch, segment, leaves, k.value, C.byref(k), None, None, None),
          "HcommGfxPlanGetTreeSegment")
    x = [None if not v else (rank_of[v] if rank_of is not None else v) for v in leaves]
    step = 1
    while step < k.value:
        for q in range(0, k.value, 2 * step):
            if x[q + step] is not None:
                x[q] = [x[q], x[q + step]]
        step *= 2
    if with_owner:  # the rank whose output takes the root, -1 = every rank's
        return x[0], off.value, nbytes.value, owner.value
    return x[0], off.value, nbytes.value


# ---- the op-base loop around a template ------------------------------------------------------------------

BUF_USER_IN, BUF_USER_OUT = 3, 4
_opbase_emit = _sig("HcommGfxOpBaseEmit", _i32, C.c_int, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp), _u64,
                    C.POINTER(_u64))
_opbase_check = _sig("HcommGfxOpBaseCheck", _i32, C.c_int, _u32, _u64, _u64, C.c_int, C.POINTER(CheckReport))
_opbase_max = _sig("HcommGfxOpBaseMaxCount", _i32, C.c_int, _u32, _u64, C.c_int, C.POINTER(_u64))
_opbase_plan = _sig("HcommGfxOpBasePlanCreate", _i32, C.c_int, C.c_int, _u32, C.POINTER(_vp), C.POINTER(_vp),
                    C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))


def opbase_emit(alg, n_ranks, count, ccl_bytes, dtype):
    n = _u64(0)
    check(_opbase_emit(alg, n_ranks, count, ccl_bytes, dtype, None, 0, C.byref(n)), "HcommGfxOpBaseEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_opbase_emit(alg, n_ranks, count, ccl_bytes, dtype, ops, n.value, C.byref(n)), "HcommGfxOpBaseEmit")
    return [ops[i].astuple() for i in range(n.value)]


def opbase_check(alg, n_ranks, count, ccl_bytes, dtype):
    rep = CheckReport()
    check(_opbase_check(alg, n_ranks, count, ccl_bytes, dtype, C.byref(rep)), "HcommGfxOpBaseCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


def opbase_max_count(alg, n_ranks, ccl_bytes, dtype):
    m = _u64(0)
    check(_opbase_max(alg, n_ranks, ccl_bytes, dtype, C.byref(m)), "HcommGfxOpBaseMaxCount")
    return m.value


class OpBasePlan(Plan):
    """HcommGfxOpBasePlanCreate: the chunked loop user buffers -> CCL buffers -> template -> user buffers."""

    def __init__(self, alg, lowering, user_in, user_out, ccl_in, ccl_out, ccl_bytes, count, dtype, op,
                 scratch_ptrs=None):
        n = len(user_in)
        self._keep = [(_vp * n)(*x) if x is not None else None for x in (user_in, user_out, ccl_in, ccl_out, scratch_ptrs)]
        p = _vp(0)
        check(_opbase_plan(alg, lowering, n, self._keep[0], self._keep[1], self._keep[2], self._keep[3], self._keep[4],
                           ccl_bytes, count, dtype, op, C.byref(p)), "HcommGfxOpBasePlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_plan_from_ops = _sig("HcommGfxPlanCreateFromOps", _i32, C.POINTER(SchedOp), _u64, _u32, C.POINTER(C.POINTER(_vp)), C.c_int,
                      C.c_int, C.POINTER(_vp))


class OpListPlan(Plan):
    """HcommGfxPlanCreateFromOps: replay a caller's own op list.  ops: tuples as schedule_emit returns them;
    buffers: {role: [pointer per rank]} for the roles the list names."""

    def __init__(self, ops, n_ranks, buffers, dtype, op):
        arr = (SchedOp * max(len(ops), 1))()
        for i, (step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes) in enumerate(ops):
            arr[i] = SchedOp(step, kind, rank, dbuf, srank, sbuf, doff, soff, nbytes)
        self._rows = [(_vp * n_ranks)(*buffers[role]) if role in buffers else None for role in range(5)]
        table = (C.POINTER(_vp) * 5)(*[C.cast(r, C.POINTER(_vp)) if r is not None else None for r in self._rows])
        p = _vp(0)
        check(_plan_from_ops(arr, len(ops), n_ranks, table, dtype, op, C.byref(p)), "HcommGfxPlanCreateFromOps")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_plan_from_ops_keep = _sig("HcommGfxPlanCreateFromOpsKeepInputs", _i32, C.POINTER(SchedOp), _u64, _u32, C.POINTER(_vp),
                           C.POINTER(_vp), C.c_int, C.c_int, C.POINTER(_vp))


class OpListKeepInputsPlan(Plan):
    """HcommGfxPlanCreateFromOpsKeepInputs: a caller's op list over the roles in / out / communication buffer as
    tree launches on in_ptrs (only read) and out_ptrs."""

    def __init__(self, ops, in_ptrs, out_ptrs, dtype, op):
        n = len(in_ptrs)
        arr = (SchedOp * max(len(ops), 1))()
        for i, (step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes) in enumerate(ops):
            arr[i] = SchedOp(step, kind, rank, dbuf, srank, sbuf, doff, soff, nbytes)
        self._in = (_vp * n)(*in_ptrs)
        self._out = (_vp * n)(*out_ptrs)
        p = _vp(0)
        check(_plan_from_ops_keep(arr, len(ops), n, self._in, self._out, dtype, op, C.byref(p)),
              "HcommGfxPlanCreateFromOpsKeepInputs")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


# ---- the ring executor's three-step allreduce over two communicator levels -------------------------------

_hier_emit = _sig("HcommGfxHierEmit", _i32, C.c_int, _u32, _u32, _u64, C.c_int, C.POINTER(SchedOp), _u64, C.POINTER(_u64))
_hier_check = _sig("HcommGfxHierCheck", _i32, C.c_int, _u32, _u32, _u64, C.c_int, C.POINTER(CheckReport))
_hier_plan = _sig("HcommGfxHierPlanCreate", _i32, C.c_int, _u32, _u32, C.POINTER(_vp), C.POINTER(_vp), _u64, C.c_int,
                  C.c_int, C.POINTER(_vp))
_mesh_emit = _sig("HcommGfxMeshHierEmit", _i32, C.c_int, _u32, _u32, _u64, C.c_int, C.POINTER(SchedOp), _u64, C.POINTER(_u64))
_mesh_check = _sig("HcommGfxMeshHierCheck", _i32, C.c_int, _u32, _u32, _u64, C.c_int, C.POINTER(CheckReport))
_mesh_plan = _sig("HcommGfxMeshHierPlanCreate", _i32, C.c_int, _u32, _u32, C.POINTER(_vp), C.POINTER(_vp), _u64, C.c_int,
                  C.c_int, C.POINTER(_vp))


def hier_emit(alg1, n_servers, n_local, count, dtype, mesh=False):
    """mesh: the mesh executor's level 0 (HcommGfxMeshHier*) instead of the ring executor's."""
    f, name = (_mesh_emit, "HcommGfxMeshHierEmit") if mesh else (_hier_emit, "HcommGfxHierEmit")
    n = _u64(0)
    check(f(alg1, n_servers, n_local, count, dtype, None, 0, C.byref(n)), name)
    ops = (SchedOp * max(n.value, 1))()
    check(f(alg1, n_servers, n_local, count, dtype, ops, n.value, C.byref(n)), name)
    return [ops[i].astuple() for i in range(n.value)]


def hier_check(alg1, n_servers, n_local, count, dtype, mesh=False):
    rep = CheckReport()
    f, name = (_mesh_check, "HcommGfxMeshHierCheck") if mesh else (_hier_check, "HcommGfxHierCheck")
    check(f(alg1, n_servers, n_local, count, dtype, C.byref(rep)), name)
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


_dbring_emit = _sig("HcommGfxDoubleRingEmit", _i32, C.c_int, _u32, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp), _u64,
                    C.POINTER(_u64))
_dbring_check = _sig("HcommGfxDoubleRingCheck", _i32, C.c_int, _u32, _u32, _u64, _u64, C.c_int, C.POINTER(CheckReport))
_dbring_plan = _sig("HcommGfxDoubleRingPlanCreate", _i32, C.c_int, _u32, _u32, C.POINTER(_vp), C.POINTER(_vp),
                    C.POINTER(_vp), C.POINTER(_vp), _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))


def dbring_emit(alg1, n_servers, n_local, count, ccl_bytes, dtype):
    n = _u64(0)
    check(_dbring_emit(alg1, n_servers, n_local, count, ccl_bytes, dtype, None, 0, C.byref(n)), "HcommGfxDoubleRingEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_dbring_emit(alg1, n_servers, n_local, count, ccl_bytes, dtype, ops, n.value, C.byref(n)), "HcommGfxDoubleRingEmit")
    return [ops[i].astuple() for i in range(n.value)]


def dbring_check(alg1, n_servers, n_local, count, ccl_bytes, dtype):
    rep = CheckReport()
    check(_dbring_check(alg1, n_servers, n_local, count, ccl_bytes, dtype, C.byref(rep)), "HcommGfxDoubleRingCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


class DoubleRingPlan(Plan):
    """HcommGfxDoubleRingPlanCreate: the double-ring allreduce executor in op-base mode, user buffers read and written
    directly."""

    def __init__(self, alg1, n_servers, n_local, user_in, user_out, ccl_in, ccl_out, ccl_bytes, count, dtype, op):
        n = n_servers * n_local
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_in, ccl_out)]
        p = _vp(0)
        check(_dbring_plan(alg1, n_servers, n_local, self._bufs[0], self._bufs[1], self._bufs[2], self._bufs[3],
                           ccl_bytes, count, dtype, op, C.byref(p)), "HcommGfxDoubleRingPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_op_emit = _sig("HcommGfxOrderPreservedEmit", _i32, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp), _u64, C.POINTER(_u64))
_op_check = _sig("HcommGfxOrderPreservedCheck", _i32, _u32, _u64, _u64, C.c_int, C.POINTER(CheckReport))
_op_plan = _sig("HcommGfxOrderPreservedPlanCreate", _i32, _u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), _u64,
                _u64, C.c_int, C.c_int, C.POINTER(_vp))


def order_preserved_emit(n_ranks, count, ccl_bytes, dtype):
    n = _u64(0)
    check(_op_emit(n_ranks, count, ccl_bytes, dtype, None, 0, C.byref(n)), "HcommGfxOrderPreservedEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_op_emit(n_ranks, count, ccl_bytes, dtype, ops, n.value, C.byref(n)), "HcommGfxOrderPreservedEmit")
    return [ops[i].astuple() for i in range(n.value)]


def order_preserved_check(n_ranks, count, ccl_bytes, dtype):
    rep = CheckReport()
    check(_op_check(n_ranks, count, ccl_bytes, dtype, C.byref(rep)), "HcommGfxOrderPreservedCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


class OrderPreservedPlan(Plan):
    """HcommGfxOrderPreservedPlanCreate: the order-preserving reduce-scatter executor on one server, op-base mode."""

    def __init__(self, user_in, user_out, ccl_out, ccl_bytes, count, dtype, op):
        n = len(user_in)
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_out)]
        p = _vp(0)
        check(_op_plan(n, self._bufs[0], self._bufs[1], self._bufs[2], ccl_bytes, count, dtype, op, C.byref(p)),
              "HcommGfxOrderPreservedPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_ops_emit = _sig("HcommGfxOrderPreservedSmallEmit", _i32, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp), _u64, C.POINTER(_u64))
_ops_check = _sig("HcommGfxOrderPreservedSmallCheck", _i32, _u32, _u64, _u64, C.c_int, C.POINTER(CheckReport))
_ops_plan = _sig("HcommGfxOrderPreservedSmallPlanCreate", _i32, _u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), _u64,
                 _u64, C.c_int, C.c_int, C.POINTER(_vp))


def order_preserved_small_emit(n_ranks, count, ccl_bytes, dtype):
    n = _u64(0)
    check(_ops_emit(n_ranks, count, ccl_bytes, dtype, None, 0, C.byref(n)), "HcommGfxOrderPreservedSmallEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_ops_emit(n_ranks, count, ccl_bytes, dtype, ops, n.value, C.byref(n)), "HcommGfxOrderPreservedSmallEmit")
    return [ops[i].astuple() for i in range(n.value)]


def order_preserved_small_check(n_ranks, count, ccl_bytes, dtype):
    rep = CheckReport()
    check(_ops_check(n_ranks, count, ccl_bytes, dtype, C.byref(rep)), "HcommGfxOrderPreservedSmallCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


class OrderPreservedSmallPlan(Plan):
    """HcommGfxOrderPreservedSmallPlanCreate: the order-preserving reduce-scatter executor's small-message branch."""

    def __init__(self, user_in, user_out, ccl_out, ccl_bytes, count, dtype, op):
        n = len(user_in)
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_out)]
        p = _vp(0)
        check(_ops_plan(n, self._bufs[0], self._bufs[1], self._bufs[2], ccl_bytes, count, dtype, op, C.byref(p)),
              "HcommGfxOrderPreservedSmallPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_opar_emit = _sig("HcommGfxOrderPreservedAllReduceEmit", _i32, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp), _u64,
                  C.POINTER(_u64))
_opar_check = _sig("HcommGfxOrderPreservedAllReduceCheck", _i32, _u32, _u64, _u64, C.c_int, C.POINTER(CheckReport))
_opar_plan = _sig("HcommGfxOrderPreservedAllReducePlanCreate", _i32, _u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                  C.POINTER(_vp), _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))


def order_preserved_ar_emit(n_ranks, count, ccl_bytes, dtype):
    n = _u64(0)
    check(_opar_emit(n_ranks, count, ccl_bytes, dtype, None, 0, C.byref(n)), "HcommGfxOrderPreservedAllReduceEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_opar_emit(n_ranks, count, ccl_bytes, dtype, ops, n.value, C.byref(n)), "HcommGfxOrderPreservedAllReduceEmit")
    return [ops[i].astuple() for i in range(n.value)]


def order_preserved_ar_check(n_ranks, count, ccl_bytes, dtype):
    rep = CheckReport()
    check(_opar_check(n_ranks, count, ccl_bytes, dtype, C.byref(rep)), "HcommGfxOrderPreservedAllReduceCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


class OrderPreservedAllReducePlan(Plan):
    """HcommGfxOrderPreservedAllReducePlanCreate: the order-preserving allreduce executor on one server, op-base mode."""

    def __init__(self, user_in, user_out, ccl_in, ccl_out, ccl_bytes, count, dtype, op):
        n = len(user_in)
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_in, ccl_out)]
        p = _vp(0)
        check(_opar_plan(n, self._bufs[0], self._bufs[1], self._bufs[2], self._bufs[3], ccl_bytes, count, dtype, op,
                         C.byref(p)), "HcommGfxOrderPreservedAllReducePlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_oph_emit = _sig("HcommGfxOrderPreservedHierAllReduceEmit", _i32, C.c_int, _u32, _u32, _u64, _u64, C.c_int,
                 C.POINTER(SchedOp), _u64, C.POINTER(_u64))
_oph_check = _sig("HcommGfxOrderPreservedHierAllReduceCheck", _i32, C.c_int, _u32, _u32, _u64, _u64, C.c_int,
                  C.POINTER(CheckReport))
_oph_plan = _sig("HcommGfxOrderPreservedHierAllReducePlanCreate", _i32, C.c_int, _u32, _u32, C.POINTER(_vp), C.POINTER(_vp),
                 C.POINTER(_vp), C.POINTER(_vp), _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))


def order_preserved_hier_ar_emit(alg1, n_servers, n_local, count, ccl_bytes, dtype):
    n = _u64(0)
    check(_oph_emit(alg1, n_servers, n_local, count, ccl_bytes, dtype, None, 0, C.byref(n)),
          "HcommGfxOrderPreservedHierAllReduceEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_oph_emit(alg1, n_servers, n_local, count, ccl_bytes, dtype, ops, n.value, C.byref(n)),
          "HcommGfxOrderPreservedHierAllReduceEmit")
    return [ops[i].astuple() for i in range(n.value)]


def order_preserved_hier_ar_check(alg1, n_servers, n_local, count, ccl_bytes, dtype):
    rep = CheckReport()
    check(_oph_check(alg1, n_servers, n_local, count, ccl_bytes, dtype, C.byref(rep)),
          "HcommGfxOrderPreservedHierAllReduceCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


class OrderPreservedHierAllReducePlan(Plan):
    """HcommGfxOrderPreservedHierAllReducePlanCreate: the order-preserving allreduce executor over two levels."""

    def __init__(self, alg1, n_servers, n_local, user_in, user_out, ccl_in, ccl_out, ccl_bytes, count, dtype, op):
        n = n_servers * n_local
        assert len(user_in) == n
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_in, ccl_out)]
        p = _vp(0)
        check(_oph_plan(alg1, n_servers, n_local, self._bufs[0], self._bufs[1], self._bufs[2], self._bufs[3], ccl_bytes,
                        count, dtype, op, C.byref(p)), "HcommGfxOrderPreservedHierAllReducePlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_ophrs_emit = _sig("HcommGfxOrderPreservedHierReduceScatterEmit", _i32, _u32, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp),
                   _u64, C.POINTER(_u64))
_ophrs_check = _sig("HcommGfxOrderPreservedHierReduceScatterCheck", _i32, _u32, _u32, _u64, _u64, C.c_int,
                    C.POINTER(CheckReport))
_ophrs_plan = _sig("HcommGfxOrderPreservedHierReduceScatterPlanCreate", _i32, _u32, _u32, C.POINTER(_vp), C.POINTER(_vp),
                   C.POINTER(_vp), C.POINTER(_vp), _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))


def order_preserved_hier_rs_emit(n_servers, n_local, count, ccl_bytes, dtype):
    n = _u64(0)
    check(_ophrs_emit(n_servers, n_local, count, ccl_bytes, dtype, None, 0, C.byref(n)),
          "HcommGfxOrderPreservedHierReduceScatterEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_ophrs_emit(n_servers, n_local, count, ccl_bytes, dtype, ops, n.value, C.byref(n)),
          "HcommGfxOrderPreservedHierReduceScatterEmit")
    return [ops[i].astuple() for i in range(n.value)]


def order_preserved_hier_rs_check(n_servers, n_local, count, ccl_bytes, dtype):
    rep = CheckReport()
    check(_ophrs_check(n_servers, n_local, count, ccl_bytes, dtype, C.byref(rep)),
          "HcommGfxOrderPreservedHierReduceScatterCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


class OrderPreservedHierReduceScatterPlan(Plan):
    """HcommGfxOrderPreservedHierReduceScatterPlanCreate: the order-preserving reduce-scatter executor over two levels."""

    def __init__(self, n_servers, n_local, user_in, user_out, ccl_out, ccl_bytes, count, dtype, op, ccl_in=None):
        """ccl_in is only needed (and used) with one device per server."""
        n = n_servers * n_local
        assert len(user_in) == n
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_out)]
        self._cin = (_vp * n)(*ccl_in) if ccl_in is not None else None
        p = _vp(0)
        check(_ophrs_plan(n_servers, n_local, self._bufs[0], self._bufs[1], self._cin, self._bufs[2], ccl_bytes, count,
                          dtype, op, C.byref(p)), "HcommGfxOrderPreservedHierReduceScatterPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_opf_plan = _sig("HcommGfxOrderPreservedFusedPlanCreate", _i32, _i32, _u32, _u32, C.POINTER(_vp), C.POINTER(_vp), _u64,
                 C.c_int, C.c_int, C.POINTER(_vp))


class OrderPreservedFusedPlan(Plan):
    """HcommGfxOrderPreservedFusedPlanCreate: either order-preserving executor as one launch on the user buffers."""

    def __init__(self, all_reduce, user_in, user_out, count, dtype, op, n_servers=1):
        n = len(user_in)
        assert n % n_servers == 0
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out)]
        p = _vp(0)
        check(_opf_plan(int(all_reduce), n_servers, n // n_servers, self._bufs[0], self._bufs[1], count, dtype, op,
                        C.byref(p)), "HcommGfxOrderPreservedFusedPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_hrs_emit = _sig("HcommGfxHierReduceScatterEmit", _i32, _i32, C.c_int, _u32, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp),
                 _u64, C.POINTER(_u64))
_hrs_check = _sig("HcommGfxHierReduceScatterCheck", _i32, _i32, C.c_int, _u32, _u32, _u64, _u64, C.c_int,
                  C.POINTER(CheckReport))
_hrs_plan = _sig("HcommGfxHierReduceScatterPlanCreate", _i32, _i32, C.c_int, _u32, _u32, C.POINTER(_vp), C.POINTER(_vp),
                 C.POINTER(_vp), C.POINTER(_vp), _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))


def hier_rs_emit(alg1, n_servers, n_local, count, ccl_bytes, dtype, mesh=False):
    n = _u64(0)
    check(_hrs_emit(int(mesh), alg1, n_servers, n_local, count, ccl_bytes, dtype, None, 0, C.byref(n)),
          "HcommGfxHierReduceScatterEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_hrs_emit(int(mesh), alg1, n_servers, n_local, count, ccl_bytes, dtype, ops, n.value, C.byref(n)),
          "HcommGfxHierReduceScatterEmit")
    return [ops[i].astuple() for i in range(n.value)]


def hier_rs_check(alg1, n_servers, n_local, count, ccl_bytes, dtype, mesh=False):
    rep = CheckReport()
    check(_hrs_check(int(mesh), alg1, n_servers, n_local, count, ccl_bytes, dtype, C.byref(rep)),
          "HcommGfxHierReduceScatterCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


class HierReduceScatterPlan(Plan):
    """HcommGfxHierReduceScatterPlanCreate: the ring (mesh=False) or mesh reduce-scatter executor over two levels."""

    def __init__(self, alg1, n_servers, n_local, user_in, user_out, ccl_in, ccl_out, ccl_bytes, count, dtype, op,
                 mesh=False):
        n = n_servers * n_local
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_in, ccl_out)]
        p = _vp(0)
        check(_hrs_plan(int(mesh), alg1, n_servers, n_local, self._bufs[0], self._bufs[1], self._bufs[2], self._bufs[3],
                        ccl_bytes, count, dtype, op, C.byref(p)), "HcommGfxHierReduceScatterPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


_dbrs_emit = _sig("HcommGfxDoubleRingReduceScatterEmit", _i32, _u32, _u64, _u64, C.c_int, C.POINTER(SchedOp), _u64,
                  C.POINTER(_u64))
_dbrs_check = _sig("HcommGfxDoubleRingReduceScatterCheck", _i32, _u32, _u64, _u64, C.c_int, C.POINTER(CheckReport))
_dbrs_plan = _sig("HcommGfxDoubleRingReduceScatterPlanCreate", _i32, _u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                  _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))


def dbring_rs_emit(n_ranks, count, ccl_bytes, dtype):
    n = _u64(0)
    check(_dbrs_emit(n_ranks, count, ccl_bytes, dtype, None, 0, C.byref(n)), "HcommGfxDoubleRingReduceScatterEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_dbrs_emit(n_ranks, count, ccl_bytes, dtype, ops, n.value, C.byref(n)), "HcommGfxDoubleRingReduceScatterEmit")
    return [ops[i].astuple() for i in range(n.value)]


def dbring_rs_check(n_ranks, count, ccl_bytes, dtype):
    rep = CheckReport()
    check(_dbrs_check(n_ranks, count, ccl_bytes, dtype, C.byref(rep)), "HcommGfxDoubleRingReduceScatterCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


_dbhrs_emit = _sig("HcommGfxDoubleRingHierReduceScatterEmit", _i32, C.c_int, C.c_int, _u32, _u32, _u32, _u64, _u64, C.c_int,
                   C.POINTER(SchedOp), _u64, C.POINTER(_u64))
_dbhrs_check = _sig("HcommGfxDoubleRingHierReduceScatterCheck", _i32, C.c_int, C.c_int, _u32, _u32, _u32, _u64, _u64, C.c_int,
                    C.POINTER(CheckReport))
_dbhrs_plan = _sig("HcommGfxDoubleRingHierReduceScatterPlanCreate", _i32, C.c_int, C.c_int, _u32, _u32, _u32, C.POINTER(_vp),
                   C.POINTER(_vp), C.POINTER(_vp), _u64, _u64, C.c_int, C.c_int, C.POINTER(_vp))
_RS_RING = 1  # HCOMM_GFX_ALG_REDUCE_SCATTER_RING


def dbring_hier_rs_emit(alg1, n_servers, n_local, count, ccl_bytes, dtype, n_pods=1, alg2=_RS_RING):
    n = _u64(0)
    check(_dbhrs_emit(alg1, alg2, n_pods, n_servers, n_local, count, ccl_bytes, dtype, None, 0, C.byref(n)),
          "HcommGfxDoubleRingHierReduceScatterEmit")
    ops = (SchedOp * max(n.value, 1))()
    check(_dbhrs_emit(alg1, alg2, n_pods, n_servers, n_local, count, ccl_bytes, dtype, ops, n.value, C.byref(n)),
          "HcommGfxDoubleRingHierReduceScatterEmit")
    return [ops[i].astuple() for i in range(n.value)]


def dbring_hier_rs_check(alg1, n_servers, n_local, count, ccl_bytes, dtype, n_pods=1, alg2=_RS_RING):
    rep = CheckReport()
    check(_dbhrs_check(alg1, alg2, n_pods, n_servers, n_local, count, ccl_bytes, dtype, C.byref(rep)),
          "HcommGfxDoubleRingHierReduceScatterCheck")
    return rep.conflicts, rep.semanticErrors, rep.message.decode()


class DoubleRingHierReduceScatterPlan(Plan):
    """HcommGfxDoubleRingHierReduceScatterPlanCreate: the double-ring reduce-scatter executor over servers and super pods."""

    def __init__(self, alg1, n_servers, n_local, user_in, user_out, ccl_in, ccl_bytes, count, dtype, op, n_pods=1,
                 alg2=_RS_RING):
        n = len(user_in)
        assert n == n_pods * n_servers * n_local
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_in)]
        p = _vp(0)
        check(_dbhrs_plan(alg1, alg2, n_pods, n_servers, n_local, self._bufs[0], self._bufs[1], self._bufs[2], ccl_bytes,
                          count, dtype, op, C.byref(p)), "HcommGfxDoubleRingHierReduceScatterPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


class DoubleRingReduceScatterPlan(Plan):
    """HcommGfxDoubleRingReduceScatterPlanCreate: the double-ring reduce-scatter executor on one server, DMA reduce."""

    def __init__(self, user_in, user_out, ccl_in, ccl_bytes, count, dtype, op):
        n = len(user_in)
        self._bufs = [(_vp * n)(*b) for b in (user_in, user_out, ccl_in)]
        p = _vp(0)
        check(_dbrs_plan(n, self._bufs[0], self._bufs[1], self._bufs[2], ccl_bytes, count, dtype, op, C.byref(p)),
              "HcommGfxDoubleRingReduceScatterPlanCreate")
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxPlanGetInfo")
        self.info = info


class HierPlan(Plan):
    """HcommGfxHierPlanCreate: ring reduce-scatter inside the servers, alg1 between them, ring all-gather inside;
    mesh=True: HcommGfxMeshHierPlanCreate, the mesh executor's multi-stream reduce-scatter and mesh all-gather."""

    def __init__(self, alg1, n_servers, n_local, in_ptrs, out_ptrs, count, dtype, op, mesh=False):
        n = n_servers * n_local
        self._in, self._out = (_vp * n)(*in_ptrs), (_vp * n)(*out_ptrs)
        p = _vp(0)
        f, name = (_mesh_plan, "HcommGfxMeshHierPlanCreate") if mesh else (_hier_plan, "HcommGfxHierPlanCreate")
        check(f(alg1, n_servers, n_local, self._in, self._out, count, dtype, op, C.byref(p)), name)
        self._p = p
        info = PlanInfo()
        check(_plan_info(self._p, C.byref(info)), "HcommGfxHierPlanGetInfo")
        self.info = info
