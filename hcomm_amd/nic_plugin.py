"""libhcomm_gfx.so bound the way the reference's plugin manager binds a NIC plugin (nic_plugin_manager.cc:113-151):
dlopen of the .so, dlsym of HcommNicPluginGetInfo / CreateEndpoint / CreateChannel, then nothing but the function
pointers of the tables they return.  ctypes mirror of include/hcomm_gfx_nic_plugin.h for the tests."""
import ctypes as C

from . import api

_vp, _i32, _u32, _u64 = C.c_void_p, C.c_int32, C.c_uint32, C.c_uint64


class CommAbiHeader(C.Structure):
    _fields_ = [("version", _u32), ("magicWord", _u32), ("size", _u32), ("reserved", _u32)]


class CommMem(C.Structure):
    _fields_ = [("type", _i32), ("addr", _vp), ("size", _u64)]


class PluginInfo(C.Structure):
    _fields_ = [("header", CommAbiHeader), ("name", C.c_char_p), ("protocolCount", _u32), ("protocols", _i32 * 4),
                ("reserved", _u64 * 8)]


def _fn(*args):
    return C.CFUNCTYPE(_i32, *args)


class EndpointOps(C.Structure):
    _fields_ = [("header", CommAbiHeader), ("init", _fn(_vp)), ("destroy", _fn(_vp)),
                ("registerMemory", _fn(_vp, _vp, C.c_char_p, _vp)), ("unregisterMemory", _fn(_vp, _vp)),
                ("memoryExport", _fn(_vp, _vp, _vp, _vp)), ("memoryImport", _fn(_vp, _vp, _u32, _vp)),
                ("memoryUnimport", _fn(_vp, _vp, _u32)), ("getListenPort", _fn(_vp, _vp))]


_copy_t = _fn(_vp, _u64, _vp, _vp, _u64)
_reduce_t = _fn(_vp, _u64, _vp, _vp, _u64, C.c_int, C.c_int)


class ChannelOps(C.Structure):
    _fields_ = [("header", CommAbiHeader), ("init", _fn(_vp)), ("destroy", _fn(_vp)), ("getStatus", _fn(_vp, _vp)),
                ("writeNbi", _fn(_vp, _vp, _vp, _u64)), ("writeNbiOnThread", _copy_t), ("writeOnThread", _copy_t),
                ("writeWithNotifyNbi", _fn(_vp, _vp, _vp, _u64, _u32)),
                ("writeWithNotifyNbiOnThread", _fn(_vp, _u64, _vp, _vp, _u64, _u32)),
                ("writeWithNotifyOnThread", _fn(_vp, _u64, _vp, _vp, _u64, _u32)),
                ("writeReduceOnThread", _reduce_t),
                ("writeReduceWithNotifyOnThread", _fn(_vp, _u64, _vp, _vp, _u64, C.c_int, C.c_int, _u32)),
                ("readNbi", _fn(_vp, _vp, _vp, _u64)), ("readNbiOnThread", _copy_t), ("readOnThread", _copy_t),
                ("readReduceOnThread", _reduce_t),
                ("notifyRecord", _fn(_vp, _u32)), ("notifyRecordOnThread", _fn(_vp, _u64, _u32)),
                ("notifyWait", _fn(_vp, _u32, _u32)), ("notifyWaitOnThread", _fn(_vp, _u64, _u32, _u32)),
                ("notifyWaitOnThreadWithDefaultTimeout", _fn(_vp, _u64, _u32)),
                ("batchTransferOnThread", _fn(_vp, _u64, _vp, _u32)),
                ("fence", _fn(_vp)), ("fenceOnThread", _fn(_vp, _u64)), ("drainOnThread", _fn(_vp, _u64))]


class ChannelDescHead(C.Structure):
    _fields_ = [("header", CommAbiHeader), ("remoteEndpoint", C.c_uint8 * 160), ("notifyNum", _u32),
                ("rest", C.c_uint8 * 180)]  # 360 bytes, as the reference's HcommChannelDesc


_so = C.CDLL(api.LIB_PATH, mode=C.RTLD_LOCAL)  # RTLD_NOW | RTLD_LOCAL in the reference; ctypes binds eagerly
_get_info = _so.HcommNicPluginGetInfo
_get_info.restype = C.POINTER(PluginInfo)
_get_info.argtypes = []
_create_ep = _so.HcommNicPluginCreateEndpoint
_create_ep.restype = _i32
_create_ep.argtypes = [_vp, C.POINTER(_vp), C.POINTER(C.POINTER(EndpointOps))]
_create_ch = _so.HcommNicPluginCreateChannel
_create_ch.restype = _i32
_create_ch.argtypes = [_vp, _vp, C.POINTER(_vp), C.POINTER(C.POINTER(ChannelOps))]


def get_info():
    return _get_info().contents


def endpoint_desc():
    return (C.c_uint8 * 160)()


def channel_desc(notify_num):
    d = ChannelDescHead()
    d.notifyNum = notify_num
    return d


def create_endpoint(desc):
    """Returns (code, ctx, ops table)."""
    ctx, ops = _vp(), C.POINTER(EndpointOps)()
    code = _create_ep(C.byref(desc) if desc is not None else None, C.byref(ctx), C.byref(ops))
    return code, ctx, (ops.contents if code == 0 else None)


def create_channel(ep_ctx, desc):
    ctx, ops = _vp(), C.POINTER(ChannelOps)()
    code = _create_ch(ep_ctx, C.byref(desc) if desc is not None else None, C.byref(ctx), C.byref(ops))
    return code, ctx, (ops.contents if code == 0 else None)
