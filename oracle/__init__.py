"""ctypes loader for the CPU oracle (oracle/hcomm_oracle.c) and the compiled reference code (oracle/_ref).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
bench.py - never by the hcomm_amd package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libhcomm_ref.so")

SUM, PROD, MAX, MIN = 0, 1, 2, 3
I8, I16, I32, F16, F32, BF16 = 0, 1, 2, 3, 4, 11
ALG_ALLREDUCE_RING, ALG_RS_RING_STAGE, ALG_ALLREDUCE_RHD, ALG_ALLREDUCE_MESH_ONESHOT, ALG_RS_MESH, \
    ALG_RS_RING_STANDALONE, ALG_ALLREDUCE_MESH_ASCENDING, ALG_ALLREDUCE_LOCAL_REDUCE, ALG_ALLREDUCE_CHUNK_MESH, \
    ALG_ALLREDUCE_NHR, ALG_RS_NHR, ALG_ALLREDUCE_NB, ALG_RS_NB, ALG_RS_LOCAL_REDUCE, ALG_ALLREDUCE_DOUBLING, \
    ALG_ALLREDUCE_NHR_ONESHOT, ALG_RS_RHD, ALG_RS_WINDOW_HALVING, ALG_ALLREDUCE_LOCAL_REDUCE_AS_WRITTEN = range(19)

# storage dtype used on the numpy side for each element type (16-bit floats travel as raw uint16)
NP_STORAGE = {I8: np.int8, I16: np.int16, I32: np.int32, F16: np.uint16, F32: np.float32, BF16: np.uint16}


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    cmd = ["make", "-C", HERE]
    if force:
        cmd.insert(1, "-B")
    subprocess.run(cmd, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


class OrcOp(C.Structure):
    _fields_ = [("step", C.c_uint32), ("kind", C.c_uint32), ("rank", C.c_uint32), ("dst_buf", C.c_uint32),
                ("src_rank", C.c_uint32), ("src_buf", C.c_uint32), ("dst_off", C.c_uint64), ("src_off", C.c_uint64),
                ("bytes", C.c_uint64)]

    def astuple(self):
        return (self.step, self.kind, self.rank, self.dst_buf, self.dst_off, self.src_rank, self.src_buf,
                self.src_off, self.bytes)


class OrcSlice(C.Structure):
    _fields_ = [("offset", C.c_uint64), ("size", C.c_uint64)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.orc_set_threads.argtypes = [C.c_int]
        L.orc_set_stride.argtypes = [C.c_uint64]
        L.orc_set_stride.restype = None
        L.orc_set_scratch.argtypes = [C.POINTER(C.c_void_p)]
        L.orc_set_scratch.restype = None
        L.orc_get_threads.restype = C.c_int
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_dtype_size.restype = C.c_uint32
        L.orc_dtype_size.argtypes = [C.c_int]
        L.orc_reduce.restype = C.c_int
        L.orc_reduce.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_int]
        L.orc_copy.restype = None
        L.orc_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64]
        L.orc_slices_ring.restype = None
        L.orc_slices_ring.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32, C.POINTER(OrcSlice)]
        L.orc_slices_rhd.restype = None
        L.orc_slices_rhd.argtypes = [C.c_uint64, C.c_uint32, C.POINTER(OrcSlice)]
        L.orc_slices_nb.restype = None
        L.orc_slices_nb.argtypes = [C.c_uint64, C.c_uint32, C.POINTER(OrcSlice)]
        L.orc_nhr_slice_map.restype = None
        L.orc_nhr_slice_map.argtypes = [C.c_uint32, C.POINTER(C.c_uint32)]
        L.orc_rs_local_reduce_scratch_bytes.restype = C.c_uint64
        L.orc_rs_local_reduce_scratch_bytes.argtypes = [C.c_uint32, C.c_uint64, C.c_int]
        L.orc_trace_opbase.restype = C.c_int64
        L.orc_trace_opbase.argtypes = [C.c_int, C.c_uint32, C.c_uint64, C.c_uint64, C.c_int, C.POINTER(OrcOp), C.c_uint64]
        L.orc_run_opbase.restype = C.c_int
        L.orc_run_opbase.argtypes = [C.c_int, C.c_uint32] + [C.POINTER(C.c_void_p)] * 4 + [C.c_uint64, C.c_uint64, C.c_int, C.c_int]
        L.orc_opbase_max_count.restype = C.c_uint64
        L.orc_opbase_max_count.argtypes = [C.c_int, C.c_uint32, C.c_uint64, C.c_int]
        L.orc_algorithmic_bytes_opbase.restype = C.c_int64
        L.orc_algorithmic_bytes_opbase.argtypes = [C.c_int, C.c_uint32, C.c_uint64, C.c_uint64, C.c_int]
        L.orc_trace_hier.restype = C.c_int64
        L.orc_trace_hier.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_uint32, C.c_uint64, C.c_int, C.POINTER(OrcOp),
                                     C.c_uint64]
        L.orc_run_hier.restype = C.c_int
        L.orc_run_hier.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_uint32, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                   C.c_uint64, C.c_int, C.c_int]
        L.orc_trace_dbring.restype = C.c_int64
        L.orc_trace_dbring.argtypes = [C.c_int, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64, C.c_int, C.POINTER(OrcOp),
                                       C.c_uint64]
        L.orc_run_dbring.restype = C.c_int
        L.orc_run_dbring.argtypes = [C.c_int, C.c_uint32, C.c_uint32] + [C.POINTER(C.c_void_p)] * 4 + \
            [C.c_uint64, C.c_uint64, C.c_int, C.c_int]
        L.orc_dbring_slices.restype = C.c_int
        L.orc_trace_order_preserved.restype = C.c_int64
        L.orc_trace_order_preserved.argtypes = [C.c_uint32, C.c_uint64, C.c_uint64, C.c_int, C.POINTER(OrcOp), C.c_uint64]
        L.orc_run_order_preserved.restype = C.c_int
        L.orc_run_order_preserved.argtypes = [C.c_uint32] + [C.POINTER(C.c_void_p)] * 4 + \
            [C.c_uint64, C.c_uint64, C.c_int, C.c_int]
        L.orc_trace_order_preserved_ar.restype = C.c_int64
        L.orc_trace_order_preserved_ar.argtypes = L.orc_trace_order_preserved.argtypes
        L.orc_run_order_preserved_ar.restype = C.c_int
        L.orc_run_order_preserved_ar.argtypes = L.orc_run_order_preserved.argtypes
        L.orc_trace_order_preserved_ar2.restype = C.c_int64
        L.orc_trace_order_preserved_ar2.argtypes = [C.c_int, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64, C.c_int,
                                                    C.POINTER(OrcOp), C.c_uint64]
        L.orc_run_order_preserved_ar2.restype = C.c_int
        L.orc_run_order_preserved_ar2.argtypes = [C.c_int, C.c_uint32, C.c_uint32] + [C.POINTER(C.c_void_p)] * 4 + \
            [C.c_uint64, C.c_uint64, C.c_int, C.c_int]
        L.orc_trace_order_preserved_rs2.restype = C.c_int64
        L.orc_trace_order_preserved_rs2.argtypes = [C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64, C.c_int,
                                                    C.POINTER(OrcOp), C.c_uint64]
        L.orc_run_order_preserved_rs2.restype = C.c_int
        L.orc_run_order_preserved_rs2.argtypes = [C.c_uint32, C.c_uint32] + [C.POINTER(C.c_void_p)] * 4 + \
            [C.c_uint64, C.c_uint64, C.c_int, C.c_int]
        L.orc_trace_order_preserved_small.restype = C.c_int64
        L.orc_trace_order_preserved_small.argtypes = L.orc_trace_order_preserved.argtypes
        L.orc_run_order_preserved_small.restype = C.c_int
        L.orc_run_order_preserved_small.argtypes = L.orc_run_order_preserved.argtypes
        L.orc_trace_hier_rs.restype = C.c_int64
        L.orc_trace_hier_rs.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64, C.c_int,
                                        C.POINTER(OrcOp), C.c_uint64]
        L.orc_run_hier_rs.restype = C.c_int
        L.orc_run_hier_rs.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_uint32] + [C.POINTER(C.c_void_p)] * 4 + \
            [C.c_uint64, C.c_uint64, C.c_int, C.c_int]
        L.orc_trace_dbring_rs.restype = C.c_int64
        L.orc_trace_dbring_rs.argtypes = [C.c_uint32, C.c_uint64, C.c_uint64, C.c_int, C.POINTER(OrcOp), C.c_uint64]
        L.orc_run_dbring_rs.restype = C.c_int
        L.orc_run_dbring_rs.argtypes = [C.c_uint32] + [C.POINTER(C.c_void_p)] * 3 + [C.c_uint64, C.c_uint64, C.c_int, C.c_int]
        L.orc_trace_dbring_rs_servers.restype = C.c_int64
        L.orc_trace_dbring_rs_servers.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64,
                                                  C.c_int, C.POINTER(OrcOp), C.c_uint64]
        L.orc_run_dbring_rs_servers.restype = C.c_int
        L.orc_run_dbring_rs_servers.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_uint32, C.c_uint32] + [C.POINTER(C.c_void_p)] * 3 + \
            [C.c_uint64, C.c_uint64, C.c_int, C.c_int]
        L.orc_trace.restype = C.c_int64
        L.orc_trace.argtypes = [C.c_int, C.c_uint32, C.c_uint64, C.c_int, C.POINTER(OrcOp), C.c_uint64]
        L.orc_run.restype = C.c_int
        L.orc_run.argtypes = [C.c_int, C.c_uint32, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_uint64, C.c_int,
                              C.c_int]
        L.orc_algorithmic_bytes.restype = C.c_int64
        L.orc_algorithmic_bytes.argtypes = [C.c_int, C.c_uint32, C.c_uint64, C.c_int]
        L.orc_reduce_k.restype = C.c_int
        L.orc_reduce_k.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.c_uint32, C.c_uint64, C.c_int, C.c_int]
        _lib = L
    return _lib


def have_ref():
    return os.path.exists(REF_PATH)


_ref = None


def ref():
    """The reference's own CPU reduce code, compiled from its sources (None when it was never built)."""
    global _ref
    if _ref is None and have_ref():
        R = C.CDLL(REF_PATH)
        for name in ("ref_mem_reduce_sum", "ref_mem_reduce_min", "ref_mem_reduce_max"):
            f = getattr(R, name)
            f.restype = None
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_int]
        R.ref_fp16_from_float.restype = C.c_uint16
        R.ref_fp16_from_float.argtypes = [C.c_float]
        R.ref_fp16_to_float.restype = C.c_float
        R.ref_fp16_to_float.argtypes = [C.c_uint16]
        for name in ("ref_fp16_add", "ref_fp16_mul"):
            f = getattr(R, name)
            f.restype = C.c_uint16
            f.argtypes = [C.c_uint16, C.c_uint16]
        for name in ("ref_fp16_gt", "ref_fp16_lt"):
            f = getattr(R, name)
            f.restype = C.c_int
            f.argtypes = [C.c_uint16, C.c_uint16]
        R.ref_fp16_from_float_n.restype = None
        R.ref_fp16_from_float_n.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64]
        R.ref_fp16_to_float_n.restype = None
        R.ref_fp16_to_float_n.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64]
        _ref = R
    return _ref


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def reduce(dst, src, dtype, op):
    """dst = dst (op) src in place on numpy arrays holding the storage type."""
    assert dst.flags.c_contiguous and src.flags.c_contiguous and dst.size == src.size
    rc = lib().orc_reduce(_ptr(dst), _ptr(src), dst.size, dtype, op)
    if rc:
        raise ValueError("orc_reduce rc=%d" % rc)
    return dst


def reduce_k(srcs, dtype, op):
    dst = np.empty_like(srcs[0])
    arr = (C.c_void_p * len(srcs))(*[s.ctypes.data for s in srcs])
    rc = lib().orc_reduce_k(_ptr(dst), arr, len(srcs), dst.size, dtype, op)
    if rc:
        raise ValueError("orc_reduce_k rc=%d" % rc)
    return dst


def slices_ring(count, unit, n):
    sl = (OrcSlice * n)()
    lib().orc_slices_ring(count, unit, n, sl)
    return [(s.offset, s.size) for s in sl]


def slices_rhd(data_bytes, block):
    sl = (OrcSlice * block)()
    lib().orc_slices_rhd(data_bytes, block, sl)
    return [(s.offset, s.size) for s in sl]


def slices_nb(total_bytes, n):
    sl = (OrcSlice * n)()
    lib().orc_slices_nb(total_bytes, n, sl)
    return [(s.offset, s.size) for s in sl]


def nhr_slice_map(n):
    m = (C.c_uint32 * n)()
    lib().orc_nhr_slice_map(n, m)
    return list(m)


def trace(alg, n, count, dtype, stride=0):
    lib().orc_set_stride(stride)
    try:
        total = lib().orc_trace(alg, n, count, dtype, None, 0)
        if total < 0:
            raise ValueError("orc_trace rc=%d" % total)
        ops = (OrcOp * max(total, 1))()
        lib().orc_trace(alg, n, count, dtype, ops, total)
    finally:
        lib().orc_set_stride(0)
    return [ops[i].astuple() for i in range(total)]


def run(alg, ins, outs, count, dtype, op, stride=0, scratch=None):
    """Execute a collective in place on lists of numpy arrays (one per rank).  stride: elements between the
    input slices of the scatter algorithms (0 = dense).  scratch: per-rank communication buffers (uint8 arrays)
    for the algorithms that stage data."""
    n = len(ins)
    a = (C.c_void_p * n)(*[x.ctypes.data for x in ins])
    b = (C.c_void_p * n)(*[x.ctypes.data for x in outs])
    sc = (C.c_void_p * n)(*[x.ctypes.data for x in scratch]) if scratch is not None else None
    lib().orc_set_stride(stride)
    lib().orc_set_scratch(sc)
    try:
        rc = lib().orc_run(alg, n, a, b, count, dtype, op)
    finally:
        lib().orc_set_stride(0)
        lib().orc_set_scratch(None)
    if rc:
        raise ValueError("orc_run rc=%d" % rc)


def algorithmic_bytes(alg, n, count, dtype):
    return lib().orc_algorithmic_bytes(alg, n, count, dtype)


# ---- the op-base loop (user buffers -> CCL buffers -> template -> user buffers) ---------------------------

def opbase_max_count(alg, n, ccl_bytes, dtype):
    return lib().orc_opbase_max_count(alg, n, ccl_bytes, dtype)


def trace_opbase(alg, n, count, ccl_bytes, dtype):
    total = lib().orc_trace_opbase(alg, n, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_opbase rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_opbase(alg, n, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_opbase(alg, user_in, user_out, ccl_in, ccl_out, count, ccl_bytes, dtype, op, scratch=None):
    """Execute the op-base loop on lists of numpy arrays (one per rank and role)."""
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in lst]) for lst in (user_in, user_out, ccl_in, ccl_out)]
    sc = (C.c_void_p * n)(*[x.ctypes.data for x in scratch]) if scratch is not None else None
    lib().orc_set_scratch(sc)
    try:
        rc = lib().orc_run_opbase(alg, n, arrs[0], arrs[1], arrs[2], arrs[3], count, ccl_bytes, dtype, op)
    finally:
        lib().orc_set_scratch(None)
    if rc:
        raise ValueError("orc_run_opbase rc=%d" % rc)


def algorithmic_bytes_opbase(alg, n, count, ccl_bytes, dtype):
    return lib().orc_algorithmic_bytes_opbase(alg, n, count, ccl_bytes, dtype)


# ---- the ring executor's three-step allreduce over two communicator levels -------------------------------

def trace_hier(alg1, n_servers, n_local, count, dtype, mesh=False):
    """mesh: the mesh executor's level 0 (multi-stream mesh reduce-scatter, mesh all-gather) instead of the ring's."""
    total = lib().orc_trace_hier(int(mesh), alg1, n_servers, n_local, count, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_hier rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_hier(int(mesh), alg1, n_servers, n_local, count, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_hier(alg1, n_servers, n_local, ins, outs, count, dtype, op, mesh=False):
    n = len(ins)
    a = (C.c_void_p * n)(*[x.ctypes.data for x in ins])
    b = (C.c_void_p * n)(*[x.ctypes.data for x in outs])
    rc = lib().orc_run_hier(int(mesh), alg1, n_servers, n_local, a, b, count, dtype, op)
    if rc:
        raise ValueError("orc_run_hier rc=%d" % rc)


# ---- the double-ring allreduce executor in op-base mode (user memory read and written directly) ----------

def trace_dbring(alg1, n_servers, n_local, count, ccl_bytes, dtype):
    total = lib().orc_trace_dbring(alg1, n_servers, n_local, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_dbring rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_dbring(alg1, n_servers, n_local, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_dbring(alg1, n_servers, n_local, user_in, user_out, ccl_in, ccl_out, count, ccl_bytes, dtype, op):
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in, ccl_out)]
    rc = lib().orc_run_dbring(alg1, n_servers, n_local, arrs[0], arrs[1], arrs[2], arrs[3], count, ccl_bytes, dtype, op)
    if rc:
        raise ValueError("orc_run_dbring rc=%d" % rc)


def dbring_slices(count, dtype, n):
    """([ring][position] -> (offset, size), [ring][position] -> device) of the double-ring slice preparation."""
    sl = (OrcSlice * (2 * n))()
    order = (C.c_uint32 * (2 * n))()
    rc = lib().orc_dbring_slices(C.c_uint64(count), dtype, C.c_uint32(n), sl, order)
    if rc:
        raise ValueError("orc_dbring_slices rc=%d" % rc)
    return ([[(sl[r * n + i].offset, sl[r * n + i].size) for i in range(n)] for r in range(2)],
            [[order[r * n + i] for i in range(n)] for r in range(2)])


# ---- the order-preserving reduce-scatter executor (plant local reduce, one server, op-base mode) ----------

def trace_order_preserved(n, count, ccl_bytes, dtype):
    total = lib().orc_trace_order_preserved(n, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_order_preserved rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_order_preserved(n, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_order_preserved(user_in, user_out, ccl_in, ccl_out, count, ccl_bytes, dtype, op):
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in, ccl_out)]
    rc = lib().orc_run_order_preserved(n, arrs[0], arrs[1], arrs[2], arrs[3], count, ccl_bytes, dtype, op)
    if rc:
        raise ValueError("orc_run_order_preserved rc=%d" % rc)


def trace_order_preserved_ar(n, count, ccl_bytes, dtype):
    """The order-preserving ALLREDUCE executor on one server: plant with borrowed space, mesh all-gather, copy out."""
    total = lib().orc_trace_order_preserved_ar(n, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_order_preserved_ar rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_order_preserved_ar(n, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_order_preserved_ar(user_in, user_out, ccl_in, ccl_out, count, ccl_bytes, dtype, op):
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in, ccl_out)]
    rc = lib().orc_run_order_preserved_ar(n, arrs[0], arrs[1], arrs[2], arrs[3], count, ccl_bytes, dtype, op)
    if rc:
        raise ValueError("orc_run_order_preserved_ar rc=%d" % rc)


def trace_order_preserved_ar2(alg1, n_servers, n_local, count, ccl_bytes, dtype):
    """The order-preserving allreduce executor over n_servers modules of n_local devices; alg1 (ALG_ALLREDUCE_RING,
    ALG_ALLREDUCE_NHR or ALG_ALLREDUCE_NB) selects the all-gather between the servers."""
    total = lib().orc_trace_order_preserved_ar2(alg1, n_servers, n_local, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_order_preserved_ar2 rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_order_preserved_ar2(alg1, n_servers, n_local, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_order_preserved_ar2(alg1, n_servers, n_local, user_in, user_out, ccl_in, ccl_out, count, ccl_bytes, dtype, op):
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in, ccl_out)]
    rc = lib().orc_run_order_preserved_ar2(alg1, n_servers, n_local, arrs[0], arrs[1], arrs[2], arrs[3], count, ccl_bytes,
                                           dtype, op)
    if rc:
        raise ValueError("orc_run_order_preserved_ar2 rc=%d" % rc)


def trace_order_preserved_rs2(n_servers, n_local, count, ccl_bytes, dtype):
    """The order-preserving reduce-scatter executor over n_servers modules of n_local devices."""
    total = lib().orc_trace_order_preserved_rs2(n_servers, n_local, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_order_preserved_rs2 rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_order_preserved_rs2(n_servers, n_local, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_order_preserved_rs2(n_servers, n_local, user_in, user_out, ccl_in, ccl_out, count, ccl_bytes, dtype, op):
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in, ccl_out)]
    rc = lib().orc_run_order_preserved_rs2(n_servers, n_local, arrs[0], arrs[1], arrs[2], arrs[3], count, ccl_bytes, dtype, op)
    if rc:
        raise ValueError("orc_run_order_preserved_rs2 rc=%d" % rc)


def trace_order_preserved_small(n, count, ccl_bytes, dtype):
    """The order-preserving reduce-scatter executor's ReduceScatterHDStage branch (4 or 8 ranks, <= 32 KiB per rank)."""
    total = lib().orc_trace_order_preserved_small(n, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_order_preserved_small rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_order_preserved_small(n, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_order_preserved_small(user_in, user_out, ccl_in, ccl_out, count, ccl_bytes, dtype, op):
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in, ccl_out)]
    rc = lib().orc_run_order_preserved_small(n, arrs[0], arrs[1], arrs[2], arrs[3], count, ccl_bytes, dtype, op)
    if rc:
        raise ValueError("orc_run_order_preserved_small rc=%d" % rc)


# ---- the ring / mesh reduce-scatter executors over two communicator levels, op-base mode -----------------

def trace_hier_rs(alg1, n_servers, n_local, count, ccl_bytes, dtype, mesh=False):
    """alg1: ALG_RS_RING_STAGE, ALG_RS_NHR, ALG_RS_NB or ALG_RS_RHD between the servers."""
    total = lib().orc_trace_hier_rs(int(mesh), alg1, n_servers, n_local, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_hier_rs rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_hier_rs(int(mesh), alg1, n_servers, n_local, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_hier_rs(alg1, n_servers, n_local, user_in, user_out, ccl_in, ccl_out, count, ccl_bytes, dtype, op, mesh=False):
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in, ccl_out)]
    rc = lib().orc_run_hier_rs(int(mesh), alg1, n_servers, n_local, arrs[0], arrs[1], arrs[2], arrs[3], count, ccl_bytes,
                               dtype, op)
    if rc:
        raise ValueError("orc_run_hier_rs rc=%d" % rc)


# ---- the double-ring reduce-scatter executor on one server, op-base mode with DMA reduce -----------------

def trace_dbring_rs(n, count, ccl_bytes, dtype):
    total = lib().orc_trace_dbring_rs(n, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_dbring_rs rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_dbring_rs(n, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_dbring_rs(user_in, user_out, ccl_in, count, ccl_bytes, dtype, op):
    n = len(user_in)
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in)]
    rc = lib().orc_run_dbring_rs(n, arrs[0], arrs[1], arrs[2], count, ccl_bytes, dtype, op)
    if rc:
        raise ValueError("orc_run_dbring_rs rc=%d" % rc)


# ---- the same executor over servers and super pods ----------------------------------------------------------

def trace_dbring_rs_servers(alg1, n_servers, n_local, count, ccl_bytes, dtype, n_pods=1, alg2=ALG_RS_RING_STAGE):
    """rank = (pod * n_servers + server) * n_local + local index; alg1 between the servers of a pod, alg2 between pods."""
    total = lib().orc_trace_dbring_rs_servers(alg1, alg2, n_pods, n_servers, n_local, count, ccl_bytes, dtype, None, 0)
    if total < 0:
        raise ValueError("orc_trace_dbring_rs_servers rc=%d" % total)
    ops = (OrcOp * max(total, 1))()
    lib().orc_trace_dbring_rs_servers(alg1, alg2, n_pods, n_servers, n_local, count, ccl_bytes, dtype, ops, total)
    return [ops[i].astuple() for i in range(total)]


def run_dbring_rs_servers(alg1, n_servers, n_local, user_in, user_out, ccl_in, count, ccl_bytes, dtype, op, n_pods=1,
                          alg2=ALG_RS_RING_STAGE):
    n = len(user_in)
    assert n == n_pods * n_servers * n_local
    arrs = [(C.c_void_p * n)(*[x.ctypes.data for x in b]) for b in (user_in, user_out, ccl_in)]
    rc = lib().orc_run_dbring_rs_servers(alg1, alg2, n_pods, n_servers, n_local, arrs[0], arrs[1], arrs[2], count, ccl_bytes,
                                         dtype, op)
    if rc:
        raise ValueError("orc_run_dbring_rs_servers rc=%d" % rc)
