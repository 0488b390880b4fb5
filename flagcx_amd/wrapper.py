"""ctypes binding of libflagcx_amd.so under FlagCX's own Python names.

Same class, method and enum names, argument order and error behaviour as the
reference's ctypes harness (plugin/interservice/flagcx_wrapper.py:170-243 for
the enums, :244-330 for the argtypes table, :520-650 for the methods), limited
to the calls of this path: communicator life cycle, the reducing and
byte-moving collectives, send / recv, group brackets.  Buffers are raw device
addresses (``tensor.data_ptr()`` for a torch tensor), ``count`` is in elements,
``stream`` is a ``flagcxStream_t`` obtained from ``adaptor_stream_create`` or
``adaptor_stream_copy``.

All ranks of a communicator live in this process on one GPU: call
``flagcxCommInitRank`` once per rank with the same unique id, then issue every
collective once per rank; the last rank's call launches it.
"""
import ctypes
from dataclasses import dataclass
from typing import Any, List, Optional

from . import _native as N
from .adaptor import load_plugin

flagcxResult_t = ctypes.c_int
flagcxDataType_t = ctypes.c_int
flagcxRedOp_t = ctypes.c_int
flagcxComm_t = ctypes.c_void_p
flagcxStream_t = ctypes.c_void_p
buffer_type = ctypes.c_void_p

FLAGCX_UNIQUE_ID_BYTES = 256


class flagcxUniqueId(ctypes.Structure):
    _fields_ = [("internal", ctypes.c_byte * FLAGCX_UNIQUE_ID_BYTES)]


class flagcxDataTypeEnum:
    flagcxInt8 = flagcxChar = 0
    flagcxUint8 = 1
    flagcxInt32 = flagcxInt = 2
    flagcxUint32 = 3
    flagcxInt64 = 4
    flagcxUint64 = 5
    flagcxFloat16 = flagcxHalf = 6
    flagcxFloat32 = flagcxFloat = 7
    flagcxFloat64 = flagcxDouble = 8
    flagcxBfloat16 = 9
    flagcxNumTypes = 10

    @classmethod
    def from_torch(cls, dtype) -> int:
        import torch
        table = {torch.int8: cls.flagcxInt8, torch.uint8: cls.flagcxUint8, torch.int32: cls.flagcxInt32,
                 torch.int64: cls.flagcxInt64, torch.float16: cls.flagcxFloat16, torch.float32: cls.flagcxFloat32,
                 torch.float64: cls.flagcxFloat64, torch.bfloat16: cls.flagcxBfloat16}
        if dtype not in table:
            raise ValueError(f"Unsupported dtype: {dtype}")
        return table[dtype]


class flagcxRedOpTypeEnum:
    flagcxSum = 0
    flagcxProd = 1
    flagcxMax = 2
    flagcxMin = 3
    flagcxAvg = 4
    flagcxNumOps = 5

    @classmethod
    def from_torch(cls, op) -> int:
        from torch.distributed import ReduceOp
        table = {ReduceOp.SUM: cls.flagcxSum, ReduceOp.PRODUCT: cls.flagcxProd, ReduceOp.MAX: cls.flagcxMax,
                 ReduceOp.MIN: cls.flagcxMin, ReduceOp.AVG: cls.flagcxAvg}
        for k, v in table.items():
            if op == k:
                return v
        raise ValueError(f"Unsupported op: {op}")


@dataclass
class Function:
    name: str
    restype: Any
    argtypes: List[Any]


class FLAGCXLibrary:
    exported_functions = [
        Function("flagcxGetErrorString", ctypes.c_char_p, [flagcxResult_t]),
        Function("flagcxGetVersion", flagcxResult_t, [ctypes.POINTER(ctypes.c_int)]),
        Function("flagcxGetUniqueId", flagcxResult_t, [ctypes.POINTER(flagcxUniqueId)]),
        Function("flagcxCommInitRank", flagcxResult_t,
                 [ctypes.POINTER(flagcxComm_t), ctypes.c_int, ctypes.POINTER(flagcxUniqueId), ctypes.c_int]),
        Function("flagcxCommDestroy", flagcxResult_t, [flagcxComm_t]),
        Function("flagcxCommCount", flagcxResult_t, [flagcxComm_t, ctypes.POINTER(ctypes.c_int)]),
        Function("flagcxCommUserRank", flagcxResult_t, [flagcxComm_t, ctypes.POINTER(ctypes.c_int)]),
        Function("flagcxBarrier", flagcxResult_t, [flagcxComm_t, flagcxStream_t]),
        Function("flagcxAllReduce", flagcxResult_t,
                 [buffer_type, buffer_type, ctypes.c_size_t, flagcxDataType_t, flagcxRedOp_t, flagcxComm_t,
                  flagcxStream_t]),
        Function("flagcxReduce", flagcxResult_t,
                 [buffer_type, buffer_type, ctypes.c_size_t, flagcxDataType_t, flagcxRedOp_t, ctypes.c_int,
                  flagcxComm_t, flagcxStream_t]),
        Function("flagcxAllGather", flagcxResult_t,
                 [buffer_type, buffer_type, ctypes.c_size_t, flagcxDataType_t, flagcxComm_t, flagcxStream_t]),
        Function("flagcxReduceScatter", flagcxResult_t,
                 [buffer_type, buffer_type, ctypes.c_size_t, flagcxDataType_t, flagcxRedOp_t, flagcxComm_t,
                  flagcxStream_t]),
        Function("flagcxSend", flagcxResult_t,
                 [buffer_type, ctypes.c_size_t, flagcxDataType_t, ctypes.c_int, flagcxComm_t, flagcxStream_t]),
        Function("flagcxRecv", flagcxResult_t,
                 [buffer_type, ctypes.c_size_t, flagcxDataType_t, ctypes.c_int, flagcxComm_t, flagcxStream_t]),
        Function("flagcxBroadcast", flagcxResult_t,
                 [buffer_type, buffer_type, ctypes.c_size_t, flagcxDataType_t, ctypes.c_int, flagcxComm_t,
                  flagcxStream_t]),
        Function("flagcxGroupStart", flagcxResult_t, [flagcxComm_t]),
        Function("flagcxGroupEnd", flagcxResult_t, [flagcxComm_t]),
    ]

    def __init__(self, so_file: Optional[str] = None):
        self.lib = ctypes.CDLL(so_file) if so_file else N.lib
        self._funcs = {}
        for func in FLAGCXLibrary.exported_functions:
            f = getattr(self.lib, func.name)
            f.restype, f.argtypes = func.restype, func.argtypes
            self._funcs[func.name] = f
        # streams come from the device-adaptor plugin, as the reference takes them from its device handle
        self.devHandle = load_plugin()

    def flagcxGetErrorString(self, result) -> str:
        return self._funcs["flagcxGetErrorString"](result).decode("utf-8")

    def FLAGCX_CHECK(self, result) -> None:
        if result != 0:
            raise RuntimeError(f"FLAGCX error: {self.flagcxGetErrorString(result)}")

    def flagcxGetVersion(self) -> str:
        version = ctypes.c_int()
        self.FLAGCX_CHECK(self._funcs["flagcxGetVersion"](ctypes.byref(version)))
        v = version.value
        return f"{v // 10000}.{v // 100 % 100}.{v % 100}"

    def flagcxGetUniqueId(self) -> flagcxUniqueId:
        unique_id = flagcxUniqueId()
        self.FLAGCX_CHECK(self._funcs["flagcxGetUniqueId"](ctypes.byref(unique_id)))
        return unique_id

    def unique_id_from_bytes(self, data: bytes) -> flagcxUniqueId:
        if len(data) != FLAGCX_UNIQUE_ID_BYTES:
            raise ValueError(f"Expected {FLAGCX_UNIQUE_ID_BYTES} bytes for flagcxUniqueId, got {len(data)} bytes")
        unique_id = flagcxUniqueId()
        ctypes.memmove(ctypes.addressof(unique_id.internal), data, FLAGCX_UNIQUE_ID_BYTES)
        return unique_id

    def flagcxCommInitRank(self, world_size: int, unique_id: flagcxUniqueId, rank: int) -> flagcxComm_t:
        comm = flagcxComm_t()
        self.FLAGCX_CHECK(self._funcs["flagcxCommInitRank"](ctypes.byref(comm), world_size, ctypes.byref(unique_id),
                                                            rank))
        return comm

    def flagcxCommDestroy(self, comm) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxCommDestroy"](comm))

    def flagcxCommCount(self, comm) -> int:
        n = ctypes.c_int()
        self.FLAGCX_CHECK(self._funcs["flagcxCommCount"](comm, ctypes.byref(n)))
        return n.value

    def flagcxCommUserRank(self, comm) -> int:
        r = ctypes.c_int()
        self.FLAGCX_CHECK(self._funcs["flagcxCommUserRank"](comm, ctypes.byref(r)))
        return r.value

    def flagcxBarrier(self, comm, stream) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxBarrier"](comm, stream))

    def flagcxAllReduce(self, sendbuff, recvbuff, count: int, datatype: int, op: int, comm, stream) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxAllReduce"](sendbuff, recvbuff, count, datatype, op, comm, stream))

    def flagcxReduce(self, sendbuff, recvbuff, count: int, datatype: int, op: int, root: int, comm, stream) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxReduce"](sendbuff, recvbuff, count, datatype, op, root, comm, stream))

    def flagcxReduceScatter(self, sendbuff, recvbuff, count: int, datatype: int, op: int, comm, stream) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxReduceScatter"](sendbuff, recvbuff, count, datatype, op, comm, stream))

    def flagcxAllGather(self, sendbuff, recvbuff, count: int, datatype: int, comm, stream) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxAllGather"](sendbuff, recvbuff, count, datatype, comm, stream))

    def flagcxSend(self, sendbuff, count: int, datatype: int, dest: int, comm, stream) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxSend"](sendbuff, count, datatype, dest, comm, stream))

    def flagcxRecv(self, recvbuff, count: int, datatype: int, src: int, comm, stream) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxRecv"](recvbuff, count, datatype, src, comm, stream))

    def flagcxBroadcast(self, sendbuff, recvbuff, count: int, datatype: int, root: int, comm, stream) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxBroadcast"](sendbuff, recvbuff, count, datatype, root, comm, stream))

    def flagcxGroupStart(self, comm) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxGroupStart"](comm))

    def flagcxGroupEnd(self, comm) -> None:
        self.FLAGCX_CHECK(self._funcs["flagcxGroupEnd"](comm))

    # ---- streams, through the device adaptor's table (flagcx_wrapper.py:877-895) ----
    def adaptor_stream_create(self):
        new_stream = flagcxStream_t()
        self.FLAGCX_CHECK(self.devHandle.streamCreate(ctypes.byref(new_stream)))
        return new_stream

    def adaptor_stream_copy(self, old_stream):
        """Wrap a foreign stream object (anything with a ``cuda_stream`` attribute
        holding the raw hipStream_t, e.g. a torch stream) or a raw handle."""
        raw = getattr(old_stream, "cuda_stream", old_stream)
        new_stream = flagcxStream_t()
        self.FLAGCX_CHECK(self.devHandle.streamCopy(ctypes.byref(new_stream), ctypes.c_void_p(raw)))
        return new_stream

    def adaptor_stream_free(self, stream) -> None:
        self.FLAGCX_CHECK(self.devHandle.streamFree(stream))

    def adaptor_stream_destroy(self, stream) -> None:
        self.FLAGCX_CHECK(self.devHandle.streamDestroy(stream))

    def adaptor_stream_synchronize(self, stream) -> None:
        self.FLAGCX_CHECK(self.devHandle.streamSynchronize(stream))
