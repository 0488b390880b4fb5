"""Load the device-adaptor plugin the way FlagCX's loader does, and offer small
helpers (device buffers, streams, events) on top of its function table.

Loader steps mirrored from flagcx/adaptor/device/device_plugin_load.cc:25-103:
dlopen(RTLD_NOW|RTLD_LOCAL) -> dlsym("flagcxDeviceAdaptorPlugin_v1") -> reject
the plugin when the name is empty or any of the 32 required pointers is NULL.
"""
import ctypes as C
import os

import numpy as np

from . import _native as N

_vp = C.c_void_p
_R = C.c_int  # flagcxResult_t


def _fn(*args):
    return C.CFUNCTYPE(_R, *args)


class DevProps(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("pciBusId", C.c_int), ("pciDeviceId", C.c_int), ("pciDomainId", C.c_int)]


LAUNCH_FUNC = C.CFUNCTYPE(None, _vp, _vp)   # flagcxLaunchFunc_t
HOST_FUNC = C.CFUNCTYPE(None, _vp)

# (name, prototype) in ABI order -- flagcx/adaptor/include/flagcx_device_adaptor.h:30-116
_V1_FIELDS = [
    ("deviceSynchronize", _fn()),
    ("deviceMemcpy", _fn(_vp, _vp, C.c_size_t, C.c_int, _vp, _vp)),
    ("deviceMemset", _fn(_vp, C.c_int, C.c_size_t, C.c_int, _vp)),
    ("deviceMalloc", _fn(C.POINTER(_vp), C.c_size_t, C.c_int, _vp)),
    ("deviceFree", _fn(_vp, C.c_int, _vp)),
    ("setDevice", _fn(C.c_int)),
    ("getDevice", _fn(C.POINTER(C.c_int))),
    ("getDeviceCount", _fn(C.POINTER(C.c_int))),
    ("getVendor", _fn(C.c_char_p)),
    ("hostGetDevicePointer", _fn(C.POINTER(_vp), _vp)),
    ("memHandleInit", _fn(C.c_int, C.POINTER(_vp))),
    ("memHandleDestroy", _fn(C.c_int, _vp)),
    ("gdrMemAlloc", _fn(C.POINTER(_vp), C.c_size_t, _vp)),
    ("gdrMemFree", _fn(_vp, _vp)),
    ("hostShareMemAlloc", _fn(C.POINTER(_vp), C.c_size_t, _vp)),
    ("hostShareMemFree", _fn(_vp, _vp)),
    ("gdrPtrMmap", _fn(C.POINTER(_vp), _vp, C.c_size_t)),
    ("gdrPtrMunmap", _fn(_vp, C.c_size_t)),
    ("streamCreate", _fn(C.POINTER(_vp))),
    ("streamDestroy", _fn(_vp)),
    ("streamCopy", _fn(C.POINTER(_vp), _vp)),
    ("streamFree", _fn(_vp)),
    ("streamSynchronize", _fn(_vp)),
    ("streamQuery", _fn(_vp)),
    ("streamWaitEvent", _fn(_vp, _vp)),
    ("streamWaitValue64", _fn(_vp, _vp, C.c_uint64, C.c_int)),
    ("streamWriteValue64", _fn(_vp, _vp, C.c_uint64, C.c_int)),
    ("eventCreate", _fn(C.POINTER(_vp), C.c_int)),
    ("eventDestroy", _fn(_vp)),
    ("eventRecord", _fn(_vp, _vp)),
    ("eventSynchronize", _fn(_vp)),
    ("eventQuery", _fn(_vp)),
    ("eventElapsedTime", _fn(C.POINTER(C.c_float), _vp, _vp)),
    ("ipcMemHandleCreate", _fn(C.POINTER(_vp), C.POINTER(C.c_size_t))),
    ("ipcMemHandleGet", _fn(_vp, _vp)),
    ("ipcMemHandleOpen", _fn(_vp, C.POINTER(_vp))),
    ("ipcMemHandleClose", _fn(_vp)),
    ("ipcMemHandleFree", _fn(_vp)),
    ("launchKernel", _fn(_vp, C.c_uint, C.c_uint, C.c_uint, C.c_uint, C.c_uint, C.c_uint, C.POINTER(_vp),
                         C.c_size_t, _vp, _vp)),
    ("copyArgsInit", _fn(C.POINTER(_vp))),
    ("copyArgsFree", _fn(_vp)),
    ("launchDeviceFunc", _fn(_vp, LAUNCH_FUNC, _vp)),
    ("getDeviceProperties", _fn(C.POINTER(DevProps), C.c_int)),
    ("getDevicePciBusId", _fn(C.c_char_p, C.c_int, C.c_int)),
    ("getDeviceByPciBusId", _fn(C.POINTER(C.c_int), C.c_char_p)),
    ("launchHostFunc", _fn(_vp, HOST_FUNC, _vp)),
    ("dmaSupport", _fn(C.POINTER(C.c_bool))),
    ("getHandleForAddressRange", _fn(_vp, _vp, C.c_size_t, C.c_ulonglong)),
]


class DeviceAdaptorV1(C.Structure):
    _fields_ = [("name", C.c_char * 32)] + _V1_FIELDS


# device_plugin_load.cc:72-88
REQUIRED = [
    "deviceSynchronize", "deviceMemcpy", "deviceMemset", "deviceMalloc", "deviceFree", "setDevice", "getDevice",
    "getDeviceCount", "getVendor", "gdrMemAlloc", "gdrMemFree", "streamCreate", "streamDestroy", "streamCopy",
    "streamFree", "streamSynchronize", "streamQuery", "streamWaitEvent", "streamWaitValue64", "streamWriteValue64",
    "eventCreate", "eventDestroy", "eventRecord", "eventSynchronize", "eventQuery", "eventElapsedTime",
    "ipcMemHandleCreate", "ipcMemHandleGet", "ipcMemHandleOpen", "ipcMemHandleClose", "ipcMemHandleFree",
    "launchHostFunc",
]
PLUGIN_SYMBOL = "flagcxDeviceAdaptorPlugin_v1"


def load_plugin(path=None):
    """Returns the plugin's function table, or raises with the loader's reason."""
    path = path or os.environ.get("FLAGCX_DEVICE_ADAPTOR_PLUGIN") or N.PLUGIN_LIB
    if not os.path.exists(path):
        raise ImportError(f"device adaptor plugin {path} is missing: run `python -m flagcx_amd.build`")
    handle = C.CDLL(path, mode=os.RTLD_NOW | os.RTLD_LOCAL)
    try:
        table = DeviceAdaptorV1.in_dll(handle, PLUGIN_SYMBOL)
    except ValueError as e:
        raise ImportError(f"symbol {PLUGIN_SYMBOL} not found in {path}") from e
    missing = [f for f in REQUIRED if not getattr(table, f)]
    if not table.name or missing:
        raise ImportError(f"plugin {path} rejected: name={table.name!r} missing={missing}")
    table._handle = handle  # keep the library mapped
    return table


class Device:
    """One GPU seen through the adaptor's function table."""

    def __init__(self, index=0, table=None):
        self.t = table or load_plugin()
        n = C.c_int(0)
        N.check(self.t.getDeviceCount(C.byref(n)), "getDeviceCount")
        if n.value <= index:
            raise RuntimeError(f"no GPU {index} (device count {n.value})")
        N.check(self.t.setDevice(index), "setDevice")
        self.index = index

    # memory -----------------------------------------------------------
    def malloc(self, nbytes, kind=N.MEM_DEVICE):
        p = _vp()
        N.check(self.t.deviceMalloc(C.byref(p), max(int(nbytes), 1), kind, None), "deviceMalloc")
        return p.value

    def free(self, ptr, kind=N.MEM_DEVICE):
        N.check(self.t.deviceFree(ptr, kind, None), "deviceFree")

    def upload(self, dptr, host: np.ndarray, stream=None):
        host = np.ascontiguousarray(host)
        N.check(self.t.deviceMemcpy(dptr, host.ctypes.data, host.nbytes, N.MEMCPY_H2D, stream, None), "H2D")

    def download(self, host: np.ndarray, dptr, stream=None):
        assert host.flags["C_CONTIGUOUS"]
        N.check(self.t.deviceMemcpy(host.ctypes.data, dptr, host.nbytes, N.MEMCPY_D2H, stream, None), "D2H")
        return host

    def copy(self, dst, src, nbytes, stream=None):
        N.check(self.t.deviceMemcpy(dst, src, nbytes, N.MEMCPY_D2D, stream, None), "D2D")

    def memset(self, dptr, value, nbytes, stream=None):
        N.check(self.t.deviceMemset(dptr, value, nbytes, N.MEM_DEVICE, stream), "memset")

    def to_device(self, host: np.ndarray):
        p = self.malloc(host.nbytes)
        self.upload(p, host)
        return p

    def to_host(self, dptr, count, np_dtype):
        return self.download(np.empty(count, dtype=np_dtype), dptr)

    # streams / events ---------------------------------------------------
    def stream_create(self):
        s = _vp()
        N.check(self.t.streamCreate(C.byref(s)), "streamCreate")
        return s.value

    def stream_destroy(self, s):
        N.check(self.t.streamDestroy(s), "streamDestroy")

    @staticmethod
    def raw_stream(s):
        """hipStream_t inside a flagcxStream_t (first member, as in FlagCX's
        AMD adaptor header)."""
        return C.cast(s, C.POINTER(_vp))[0] if s else None

    def stream_sync(self, s):
        N.check(self.t.streamSynchronize(s), "streamSynchronize")

    def sync(self):
        N.check(self.t.deviceSynchronize(), "deviceSynchronize")

    def set_device(self):
        """Make this GPU current for the calling host thread."""
        N.check(self.t.setDevice(self.index), "setDevice")

    def event_create(self, timing=True):
        e = _vp()
        N.check(self.t.eventCreate(C.byref(e), 0 if timing else 1), "eventCreate")
        return e.value

    def event_record(self, e, s):
        N.check(self.t.eventRecord(e, s), "eventRecord")

    def event_sync(self, e):
        N.check(self.t.eventSynchronize(e), "eventSynchronize")

    def event_ms(self, a, b):
        ms = C.c_float(0)
        N.check(self.t.eventElapsedTime(C.byref(ms), a, b), "eventElapsedTime")
        return ms.value

    def event_destroy(self, e):
        N.check(self.t.eventDestroy(e), "eventDestroy")
