"""ctypes binding of libhcomm_caller.so (hcomm_amd/csrc/hg_caller.c): a stand-in for the operator library that CALLS
the primitives.  It binds libhcomm_gfx.so by the reference's symbol names and replays whole schedules through
HcommBatchModeStart / HcommLocal{Copy,Reduce}OnThread / HcommBatchModeEnd, or eagerly on one thread per rank with
notifies between the steps.  Used by bench.py and the GPU tests; the library itself knows nothing of it."""
import ctypes as C
import os

from . import api

CALLER_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libhcomm_caller.so")
if not os.path.exists(CALLER_PATH):
    raise ImportError("libhcomm_caller.so is not built (%s); run `make -C hcomm_amd/csrc`" % CALLER_PATH)
_lib = C.CDLL(CALLER_PATH)


class CallerStats(C.Structure):
    _fields_ = [("batches", C.c_uint32), ("calls", C.c_uint32), ("notifies", C.c_uint32), ("reserved", C.c_uint32),
                ("host_us", C.c_double), ("host_us_end", C.c_double), ("host_us_end_max", C.c_double),
                ("host_us_notify", C.c_double)]


_vpp = C.POINTER(C.c_void_p)
_lib.hg_caller_bind.restype = C.c_int
_lib.hg_caller_bind.argtypes = [C.c_char_p]
_lib.hg_caller_replay_batched.restype = C.c_int32
_lib.hg_caller_replay_batched.argtypes = [C.c_uint64, C.POINTER(api.SchedOp), C.c_uint64, C.POINTER(_vpp), C.c_int,
                                          C.c_int, C.POINTER(CallerStats)]
_lib.hg_caller_replay_one_batch.restype = C.c_int32
_lib.hg_caller_replay_one_batch.argtypes = _lib.hg_caller_replay_batched.argtypes
_lib.hg_caller_replay_threads.restype = C.c_int32
_lib.hg_caller_replay_threads.argtypes = [C.POINTER(C.c_uint64), C.c_uint32, C.POINTER(api.SchedOp), C.c_uint64,
                                          C.POINTER(_vpp), C.c_int, C.c_int, C.c_uint32, C.POINTER(CallerStats)]
_lib.hg_caller_replay_host_threads.restype = C.c_int32
_lib.hg_caller_replay_host_threads.argtypes = _lib.hg_caller_replay_threads.argtypes
_lib.hg_caller_replay_threads_batched.restype = C.c_int32
_lib.hg_caller_replay_threads_batched.argtypes = _lib.hg_caller_replay_threads.argtypes
_lib.hg_caller_pool_shutdown.restype = None
if _lib.hg_caller_bind(api.LIB_PATH.encode()) != 0:
    raise ImportError("libhcomm_caller.so could not bind the primitives of %s" % api.LIB_PATH)


def pool_shutdown():
    """Stop the host threads that run_on_host_threads keeps between calls."""
    _lib.hg_caller_pool_shutdown()


class Replay:
    """A schedule (the records of HcommGfxScheduleEmit, or any list of (step, kind, rank, dstBuf, dstOff, srcRank,
    srcBuf, srcOff, bytes) tuples ordered by step) bound to rank buffers: bufs = {role: [address per rank]} with role
    0 = in, 1 = out, 2 = communication buffer."""

    def __init__(self, ops, bufs, dtype, op):
        self.n = len(ops)
        self._ops = (api.SchedOp * max(self.n, 1))()
        for i, (step, kind, rank, dbuf, doff, srank, sbuf, soff, nbytes) in enumerate(ops):
            o = self._ops[i]
            o.step, o.kind, o.rank, o.dstBuf, o.dstOff = step, kind, rank, dbuf, doff
            o.srcRank, o.srcBuf, o.srcOff, o.bytes = srank, sbuf, soff, nbytes
        self._rows = {}
        self._bufs = (_vpp * 5)()
        for role, ptrs in bufs.items():
            row = (C.c_void_p * len(ptrs))(*ptrs)
            self._rows[role] = row
            self._bufs[role] = C.cast(row, _vpp)
        self.dtype, self.op = dtype, op
        self.steps = len(set(o[0] for o in ops))

    def run_batched(self, thread):
        """One HcommBatchModeStart / End pair per step on one thread.  Returns (code, CallerStats)."""
        st = CallerStats()
        code = _lib.hg_caller_replay_batched(thread, self._ops, self.n, self._bufs, self.dtype, self.op, C.byref(st))
        return code, st

    def run_one_batch(self, thread):
        """The whole list between ONE HcommBatchModeStart / End pair on one thread.  Returns (code, CallerStats)."""
        st = CallerStats()
        code = _lib.hg_caller_replay_one_batch(thread, self._ops, self.n, self._bufs, self.dtype, self.op, C.byref(st))
        return code, st

    def run_on_threads(self, threads, timeout=10):
        """Rank r's operations on threads[r], eagerly, with notifies between the steps (threads need one notify slot
        per rank).  Returns (code, CallerStats)."""
        arr = (C.c_uint64 * len(threads))(*threads)
        st = CallerStats()
        code = _lib.hg_caller_replay_threads(arr, len(threads), self._ops, self.n, self._bufs, self.dtype, self.op,
                                             timeout, C.byref(st))
        return code, st

    def run_on_threads_batched(self, threads, timeout=10):
        """The calls of run_on_threads between one HcommBatchModeStart / End pair: the collective as one batch over all
        its threads.  host_us_end of the returned stats is the time inside HcommBatchModeEnd."""
        arr = (C.c_uint64 * len(threads))(*threads)
        st = CallerStats()
        code = _lib.hg_caller_replay_threads_batched(arr, len(threads), self._ops, self.n, self._bufs, self.dtype,
                                                     self.op, timeout, C.byref(st))
        return code, st

    def run_on_host_threads(self, threads, timeout=10):
        """As run_on_threads, with rank r's calls issued by a host thread of its own (a pool kept between calls):
        host_us_end_max of the returned stats is the slowest worker's host time."""
        arr = (C.c_uint64 * len(threads))(*threads)
        st = CallerStats()
        code = _lib.hg_caller_replay_host_threads(arr, len(threads), self._ops, self.n, self._bufs, self.dtype, self.op,
                                                  timeout, C.byref(st))
        return code, st
