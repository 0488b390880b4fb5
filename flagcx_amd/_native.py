"""ctypes bindings of include/flagcx_amd/fx_kernels.h and fx_synth.h."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# FLAGCX_AMD_LIB_DIR points at another build of the libraries (A/B measurements)
LIB_DIR = os.environ.get("FLAGCX_AMD_LIB_DIR") or os.path.join(_HERE, "lib")
KERNEL_LIB = os.path.join(LIB_DIR, "libflagcx_amd.so")
PLUGIN_LIB = os.path.join(LIB_DIR, "libflagcx-device-mi355x.so")

# FlagCX enum values (flagcx/include/flagcx.h:21-66)
SUCCESS, DEVICE_ERROR, SYSTEM_ERROR, INTERNAL_ERROR, INVALID_ARGUMENT = 0, 1, 2, 3, 4
INVALID_USAGE, IN_PROGRESS, NOT_SUPPORTED = 5, 7, 9
DT_INT8, DT_UINT8, DT_INT32, DT_UINT32, DT_INT64, DT_UINT64 = 0, 1, 2, 3, 4, 5
DT_FP16, DT_FP32, DT_FP64, DT_BF16 = 6, 7, 8, 9
OP_SUM, OP_PROD, OP_MAX, OP_MIN, OP_AVG = 0, 1, 2, 3, 4
MEMCPY_H2D, MEMCPY_D2H, MEMCPY_D2D = 0, 1, 2
MEM_HOST, MEM_DEVICE, MEM_MANAGED = 0, 1, 2
# TIMER_COLL_* slots of fxHostStagedAllReduce (include/flagcx_amd/fx_host_staged.h)
TIMER_NAMES = ("total", "calc", "comm", "mem", "mem_d2h", "mem_h2d", "alloc", "free")
STATIC_MAX_SLICES = 1024   # FX_STATIC_MAX_SLICES of include/flagcx_amd/fx_kernels.h

DTYPE_SIZE = {DT_INT8: 1, DT_UINT8: 1, DT_INT32: 4, DT_UINT32: 4, DT_INT64: 8, DT_UINT64: 8,
              DT_FP16: 2, DT_FP32: 4, DT_FP64: 8, DT_BF16: 2}
# host-side container dtypes: 16-bit floats travel as raw uint16 bit patterns
NP_DTYPE = {DT_INT8: np.int8, DT_UINT8: np.uint8, DT_INT32: np.int32, DT_UINT32: np.uint32, DT_INT64: np.int64,
            DT_UINT64: np.uint64, DT_FP16: np.uint16, DT_FP32: np.float32, DT_FP64: np.float64, DT_BF16: np.uint16}


class FlagcxError(RuntimeError):
    def __init__(self, code, what=""):
        super().__init__(f"flagcxResult_t={code} {what}")
        self.code = code


def check(rc, what=""):
    if rc != SUCCESS:
        raise FlagcxError(rc, what)
    return rc


class ReduceTrigger(C.Structure):
    _fields_ = [("value", C.c_uint64 * 4)]


class BcastDesc(C.Structure):
    _fields_ = [("inp", C.c_void_p * 8), ("out", C.c_void_p * 8), ("count", C.c_uint64)]


class Chunk(C.Structure):
    _fields_ = [("in_off", C.c_uint64), ("out_off", C.c_uint64), ("count", C.c_uint64),
                ("first", C.c_int), ("in_sel", C.c_int), ("out_sel", C.c_int)]


class SliceDesc(C.Structure):
    _fields_ = [("in_", C.c_void_p * 8), ("out", C.c_void_p), ("count", C.c_uint64)]


def _load(path):
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m flagcx_amd.build` "
            "(hipcc, gfx950). There is no CPU fallback.")
    return C.CDLL(path, mode=C.RTLD_GLOBAL)


lib = _load(KERNEL_LIB)

_vp, _sz, _i = C.c_void_p, C.c_size_t, C.c_int
_SIGS = {
    "fx_reduce_copy": (_i, [_vp, C.POINTER(_vp), _i, _sz, _i, _i, _i, _vp]),
    "fx_reduce2": (_i, [_vp, _vp, _vp, _sz, _i, _i, _vp]),
    "fx_trigger_set": (None, [C.POINTER(ReduceTrigger), C.c_uint64, C.c_uint64, C.c_uint64, _sz, _sz, _i, _i, _i]),
    "fx_trigger_get": (None, [C.POINTER(ReduceTrigger)] + [C.POINTER(C.c_uint64)] * 5 + [C.POINTER(_i)] * 3),
    "fx_reduce_triggers": (_i, [C.POINTER(ReduceTrigger), _sz, _vp]),
    "fx_reduce_slices": (_i, [C.POINTER(SliceDesc), _sz, _i, _i, _i, _vp]),
    "fx_reduce_bcast_slices": (_i, [C.POINTER(BcastDesc), _sz, _i, _i, _i, _i, _vp]),
    "fx_reduce_ordered": (_i, [C.POINTER(BcastDesc), _sz, _i, _i, _i, _i, _i, _vp]),
    "fx_copy_slices": (_i, [C.POINTER(SliceDesc), _sz, _vp]),
    "fx_reduce_bcast": (_i, [C.POINTER(_vp), _i, C.POINTER(_vp), _i, _sz, _i, _i, _i, _vp]),
    "fx_reduce_chunks": (_i, [C.POINTER(_vp), _i, C.POINTER(_vp), _i, C.POINTER(Chunk), _i, _i, _i, _vp]),
    "fx_alltoall": (_i, [C.POINTER(_vp), C.POINTER(_vp), _i, _sz, _vp]),
    "fx_plan_create": (_i, [C.POINTER(_vp), C.POINTER(SliceDesc), _sz, _i, _i, _i]),
    "fx_plan_launch": (_i, [_vp, _vp]),
    "fx_plan_destroy": (_i, [_vp]),
    "fx_reduce_slices_static": (_i, [C.POINTER(SliceDesc), _sz, _i, _i, _i, _vp]),
    "fx_pack": (_i, [_vp, _vp, C.POINTER(_sz), C.POINTER(_sz), _i, _i, _vp]),
    "fx_unpack": (_i, [_vp, _vp, C.POINTER(_sz), C.POINTER(_sz), _i, _i, _vp]),
    "fx_fifo_bytes": (_sz, [_sz]),
    "fx_fifo_init": (_i, [_vp, _sz]),
    "fx_fifo_enqueue": (_i, [_vp, C.c_uint64, C.c_uint64, C.c_uint64, _sz, _sz, _i, _i, C.POINTER(_i)]),
    "fx_fifo_poll_state": (_i, [_vp, _i]),
    "fx_fifo_set_state": (_i, [_vp, _i, _i]),
    "fx_fifo_terminate": (_i, [_vp]),
    "fx_fifo_run_batch": (_i, [_vp, _vp, _sz, C.c_ulonglong]),
    "fx_fifo_consumer_create": (_i, [C.POINTER(_vp), _sz]),
    "fx_fifo_consumer_launch": (_i, [_vp, _vp, _vp, C.c_ulonglong, _vp]),
    "fx_fifo_consumer_status": (_i, [_vp, C.POINTER(_i), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "fx_fifo_consumer_destroy": (_i, [_vp]),
    "fx_dtype_size": (_sz, [_i]),
    "fx_split": (None, [_sz, _sz, _sz, C.POINTER(_sz), C.POINTER(_sz)]),
    "fx_nredslices": (_sz, [_sz, _i, _sz, _sz, _sz]),
    "fx_version": (C.c_char_p, []),
    "fx_synth_fill": (_i, [_vp, _sz, _i, _i, C.c_double, C.c_double, C.c_uint64, C.c_uint64, _i]),
}
class RedNode(C.Structure):
    _fields_ = [("step", C.c_int32), ("rank", C.c_int32), ("in1_buf", C.c_int32), ("in2_buf", C.c_int32),
                ("out_buf", C.c_int32), ("slice", C.c_int32), ("in1_off", C.c_uint64), ("in2_off", C.c_uint64),
                ("out_off", C.c_uint64), ("count", C.c_uint64)]


_szp = C.POINTER(_sz)
_SIGS.update({
    # include/flagcx_amd/fx_sim.h
    "fxSimCommInitAll": (_i, [C.POINTER(_vp), _i]),
    "fxSimCommDestroyAll": (_i, [C.POINTER(_vp), _i]),
    "fxSimCommConfig": (_i, [_vp, _i, C.c_longlong]),
    "fxSimCommProgress": (_i, [_vp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "fxSimRegisterWindows": (_i, [_vp, C.POINTER(_vp), _sz]),
    "fxSimCommInitRank": (_i, [C.POINTER(_vp), _i, _vp, _sz, _i]),
    "fxSimCommDestroy": (_i, [_vp]),
    "fxSimCommDevice": (_i, [_vp, C.POINTER(_i)]),
    "flagcxGetVersion": (_i, [C.POINTER(_i)]),
    "flagcxGetUniqueId": (_i, [_vp]),
    "flagcxCommInitRank": (_i, [C.POINTER(_vp), _i, _vp, _i]),
    "flagcxCommDestroy": (_i, [_vp]),
    "flagcxGetErrorString": (C.c_char_p, [_i]),
    "flagcxBarrier": (_i, [_vp, _vp]),
    "flagcxGather": (_i, [_vp, _vp, _sz, _i, _i, _vp, _vp]),
    "flagcxScatter": (_i, [_vp, _vp, _sz, _i, _i, _vp, _vp]),
    "flagcxBroadcast": (_i, [_vp, _vp, _sz, _i, _i, _vp, _vp]),
    "flagcxAlltoAll": (_i, [_vp, _vp, _sz, _i, _vp, _vp]),
    "flagcxSend": (_i, [_vp, _sz, _i, _i, _vp, _vp]),
    "flagcxRecv": (_i, [_vp, _sz, _i, _i, _vp, _vp]),
    "flagcxGroupStart": (_i, [_vp]),
    "flagcxGroupEnd": (_i, [_vp]),
    "flagcxCommCount": (_i, [_vp, C.POINTER(_i)]),
    # fx_handle.h: what an application calls around the collectives
    "flagcxDeviceHandleInit": (_i, [C.POINTER(_vp)]),
    "flagcxDeviceHandleFree": (_i, [_vp]),
    "flagcxHandleInit": (_i, [C.POINTER(_vp)]),
    "flagcxHandleFree": (_i, [_vp]),
    "flagcxMemAlloc": (_i, [C.POINTER(_vp), _sz, _i]),
    "flagcxMemFree": (_i, [_vp, _i]),
    "flagcxCommRegister": (_i, [_vp, _vp, _sz, C.POINTER(_vp), _i]),
    "flagcxCommDeregister": (_i, [_vp, _vp, _i]),
    "flagcxCommWindowRegister": (_i, [_vp, _vp, _sz, C.POINTER(_vp), _i, _i]),
    "flagcxCommWindowDeregister": (_i, [_vp, _vp, _i]),
    "flagcxIsHomoComm": (_i, [_vp, C.POINTER(_i)]),
    "flagcxCommFinalize": (_i, [_vp]),
    "flagcxCommAbort": (_i, [_vp]),
    "flagcxCommResume": (_i, [_vp]),
    "flagcxCommSuspend": (_i, [_vp]),
    "flagcxGetLastError": (C.c_char_p, [_vp]),
    "flagcxCommGetAsyncError": (_i, [_vp, C.POINTER(_i)]),
    "flagcxCommGetDeviceNumber": (_i, [_vp, C.POINTER(_i)]),
    "flagcxCommUserRank": (_i, [_vp, C.POINTER(_i)]),
    "flagcxReduce": (_i, [_vp, _vp, _sz, _i, _i, _i, _vp, _vp]),
    "flagcxAllReduce": (_i, [_vp, _vp, _sz, _i, _i, _vp, _vp]),
    "flagcxReduceScatter": (_i, [_vp, _vp, _sz, _i, _i, _vp, _vp]),
    "flagcxAllGather": (_i, [_vp, _vp, _sz, _i, _vp, _vp]),
    "flagcxAlltoAllv": (_i, [_vp, _szp, _szp, _vp, _szp, _szp, _i, _vp, _vp]),
    "flagcxCustomAllReduceImpl": (_i, [_vp, _vp, _sz, _i, _i, _vp, _vp]),
    # include/flagcx_amd/fx_host_staged.h
    "fxHostStagedCreate": (_i, [C.POINTER(_vp), _i, _vp]),
    "fxHostStagedAllReduce": (_i, [_vp, C.POINTER(_vp), C.POINTER(_vp), _sz, _i, _i, C.POINTER(C.c_uint64)]),
    "fxHostStagedReduce": (_i, [_vp, C.POINTER(_vp), C.POINTER(_vp), _sz, _i, _i, _i, C.POINTER(C.c_uint64)]),
    "fxHostStagedReduceScatter": (_i, [_vp, C.POINTER(_vp), C.POINTER(_vp), _sz, _i, _i, C.POINTER(C.c_uint64)]),
    "fxHostStagedDestroy": (_i, [_vp]),
    "fx_part_ring_ar": (_sz, [_sz, _i, _i, _sz, _sz, C.POINTER(RedNode)]),
    "fx_part_ring_rs": (_sz, [_sz, _i, _i, _sz, _sz, C.POINTER(RedNode)]),
    "fx_part_locred": (_sz, [_sz, _i, _i, _sz, C.POINTER(RedNode)]),
})
for _name, (_res, _args) in _SIGS.items():
    _f = getattr(lib, _name)
    _f.restype, _f.argtypes = _res, _args


def exported_symbols():
    """Names this binding expects from libflagcx_amd.so (the C-ABI surface)."""
    return sorted(_SIGS)
