"""Load the CCL-adaptor plugin the way FlagCX's loader does
(flagcx/adaptor/ccl/ccl_plugin_load.cc:22-101): dlopen, dlsym
"flagcxCCLAdaptorPlugin_v1", reject it when the name or any of the 34 function
pointers is NULL."""
import ctypes as C
import os

from . import _native as N

_vp, _sz, _i, _R = C.c_void_p, C.c_size_t, C.c_int, C.c_int
_szp = C.POINTER(C.c_size_t)
CCL_PLUGIN_LIB = os.path.join(N.LIB_DIR, "libflagcx-ccl-mi355x.so")
UNIQUE_ID_BYTES = 4120


def _fn(*args, res=_R):
    return C.CFUNCTYPE(res, *args)


_FIELDS = [
    ("getVersion", _fn(C.POINTER(_i))),
    ("getUniqueId", _fn(C.POINTER(_vp))),
    ("getErrorString", _fn(_i, res=C.c_char_p)),
    ("getLastError", _fn(_vp, res=C.c_char_p)),
    ("getStagedBuffer", _fn(_vp, C.POINTER(_vp), _sz, _i)),
    ("commInitRank", _fn(C.POINTER(_vp), _i, _vp, _i, _vp)),
    ("commFinalize", _fn(_vp)),
    ("commDestroy", _fn(_vp)),
    ("commAbort", _fn(_vp)),
    ("commResume", _fn(_vp)),
    ("commSuspend", _fn(_vp)),
    ("commCount", _fn(_vp, C.POINTER(_i))),
    ("commGetDeviceNumber", _fn(_vp, C.POINTER(_i))),
    ("commUserRank", _fn(_vp, C.POINTER(_i))),
    ("commGetAsyncError", _fn(_vp, C.POINTER(_i))),
    ("memAlloc", _fn(C.POINTER(_vp), _sz)),
    ("memFree", _fn(_vp)),
    ("commRegister", _fn(_vp, _vp, _sz, C.POINTER(_vp))),
    ("commDeregister", _fn(_vp, _vp)),
    ("commWindowRegister", _fn(_vp, _vp, _sz, C.POINTER(_vp), _i)),
    ("commWindowDeregister", _fn(_vp, _vp)),
    ("reduce", _fn(_vp, _vp, _sz, _i, _i, _i, _vp, _vp)),
    ("gather", _fn(_vp, _vp, _sz, _i, _i, _vp, _vp)),
    ("scatter", _fn(_vp, _vp, _sz, _i, _i, _vp, _vp)),
    ("broadcast", _fn(_vp, _vp, _sz, _i, _i, _vp, _vp)),
    ("allReduce", _fn(_vp, _vp, _sz, _i, _i, _vp, _vp)),
    ("reduceScatter", _fn(_vp, _vp, _sz, _i, _i, _vp, _vp)),
    ("allGather", _fn(_vp, _vp, _sz, _i, _vp, _vp)),
    ("alltoAll", _fn(_vp, _vp, _sz, _i, _vp, _vp)),
    ("alltoAllv", _fn(_vp, _szp, _szp, _vp, _szp, _szp, _i, _vp, _vp)),
    ("send", _fn(_vp, _sz, _i, _i, _vp, _vp)),
    ("recv", _fn(_vp, _sz, _i, _i, _vp, _vp)),
    ("groupStart", _fn()),
    ("groupEnd", _fn()),
]


class CCLAdaptorV1(C.Structure):
    _fields_ = [("name", C.c_char_p)] + _FIELDS


PLUGIN_SYMBOL = "flagcxCCLAdaptorPlugin_v1"


def load_plugin(path=None):
    path = path or os.environ.get("FLAGCX_CCL_ADAPTOR_PLUGIN") or CCL_PLUGIN_LIB
    if not os.path.exists(path):
        raise ImportError(f"CCL adaptor plugin {path} is missing: run `python -m flagcx_amd.build`")
    handle = C.CDLL(path, mode=os.RTLD_NOW | os.RTLD_LOCAL)
    try:
        table = CCLAdaptorV1.in_dll(handle, PLUGIN_SYMBOL)
    except ValueError as e:
        raise ImportError(f"symbol {PLUGIN_SYMBOL} not found in {path}") from e
    missing = [f for f, _ in _FIELDS if not getattr(table, f)]
    if not table.name or missing:
        raise ImportError(f"plugin {path} rejected: name={table.name!r} missing={missing}")
    table._handle = handle
    return table
