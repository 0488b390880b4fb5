"""Communicators joined rank by rank from a unique id, over the C entry points
of include/flagcx_amd/fx_sim.h (whose names and argument lists are FlagCX's own,
flagcx/include/flagcx.h:282-484).

Every rank of a communicator lives in this process on one GPU.  A ``Rank`` is
one communicator handle; a collective is complete once every rank of the group
has posted it, and the last post enqueues the work:

    ranks = join(4)                       # or Rank.from_id(id_bytes, 4, r) rank by rank
    for r in ranks:
        r.all_reduce(send[r.index], recv[r.index], count, N.DT_BF16, N.OP_SUM, stream)

Buffers are raw device addresses (``tensor.data_ptr()`` for a torch tensor),
counts are elements, ``stream`` is a flagcxStream_t handle (``Device.stream_create``
or ``borrow_stream`` around a foreign hipStream_t).  A failing call raises
``N.FlagcxError`` carrying the flagcxResult_t code and the library's text for it.
"""
import ctypes as C

from . import _native as N
from .adaptor import load_plugin

lib = N.lib
ID_BYTES = 256            # FLAGCX_UNIQUE_ID_BYTES, include/flagcx_amd/fx_types.h

# torch dtype / ReduceOp names -> FlagCX codes; looked up by name so that this
# module does not import torch.
_DTYPE_BY_NAME = {"int8": N.DT_INT8, "uint8": N.DT_UINT8, "int32": N.DT_INT32, "int64": N.DT_INT64,
                  "float16": N.DT_FP16, "float32": N.DT_FP32, "float64": N.DT_FP64, "bfloat16": N.DT_BF16,
                  "uint32": N.DT_UINT32, "uint64": N.DT_UINT64}
_OP_BY_NAME = {"SUM": N.OP_SUM, "PRODUCT": N.OP_PROD, "MAX": N.OP_MAX, "MIN": N.OP_MIN, "AVG": N.OP_AVG}


def dtype_code(torch_dtype):
    """FlagCX datatype of a torch dtype (``torch.bfloat16`` -> 9)."""
    name = str(torch_dtype).rsplit(".", 1)[-1]
    try:
        return _DTYPE_BY_NAME[name]
    except KeyError:
        raise TypeError(f"{torch_dtype} has no FlagCX datatype") from None


def op_code(reduce_op):
    """FlagCX reduction of a ``torch.distributed.ReduceOp`` member."""
    name = (getattr(reduce_op, "name", None) or str(reduce_op)).rsplit(".", 1)[-1].upper()
    try:
        return _OP_BY_NAME[name]
    except KeyError:
        raise TypeError(f"{reduce_op} has no FlagCX reduction") from None


def error_text(code):
    return lib.flagcxGetErrorString(code).decode()


def _ok(code, what):
    if code != N.SUCCESS:
        raise N.FlagcxError(code, f"{what}: {error_text(code)}")


def version():
    """(major, minor, patch) of the library."""
    v = C.c_int()
    _ok(lib.flagcxGetVersion(C.byref(v)), "flagcxGetVersion")
    return v.value // 10000, v.value // 100 % 100, v.value % 100


def new_id():
    """A fresh unique id as 256 bytes, ready to be handed to the other ranks."""
    buf = C.create_string_buffer(ID_BYTES)
    _ok(lib.flagcxGetUniqueId(buf), "flagcxGetUniqueId")
    return buf.raw


def borrow_stream(raw, table=None):
    """flagcxStream_t around a foreign hipStream_t (an integer, or an object with a
    ``cuda_stream`` attribute such as a torch stream).  The handle does not own
    the stream; release it with ``return_stream``."""
    t = table or load_plugin()
    h = C.c_void_p()
    _ok(t.streamCopy(C.byref(h), C.c_void_p(getattr(raw, "cuda_stream", raw))), "streamCopy")
    return h.value


def return_stream(handle, table=None):
    _ok((table or load_plugin()).streamFree(handle), "streamFree")


class Rank:
    """One rank's communicator."""

    def __init__(self, handle, index, size):
        self.handle, self.index, self.size = handle, index, size

    @classmethod
    def from_id(cls, id_bytes, size, index):
        if len(id_bytes) != ID_BYTES:
            raise ValueError(f"a unique id is {ID_BYTES} bytes, not {len(id_bytes)}")
        h = C.c_void_p()
        _ok(lib.flagcxCommInitRank(C.byref(h), size, C.create_string_buffer(bytes(id_bytes), ID_BYTES), index),
            "flagcxCommInitRank")
        return cls(h, index, size)

    def close(self):
        if self.handle is not None:
            _ok(lib.flagcxCommDestroy(self.handle), "flagcxCommDestroy")
            self.handle = None

    def reported(self):
        """(rank, size) as the library reports them for this handle."""
        r, n = C.c_int(), C.c_int()
        _ok(lib.flagcxCommUserRank(self.handle, C.byref(r)), "flagcxCommUserRank")
        _ok(lib.flagcxCommCount(self.handle, C.byref(n)), "flagcxCommCount")
        return r.value, n.value

    # -- collectives: arguments in the order of the C prototypes, minus the communicator --
    def all_reduce(self, send, recv, count, dtype, op, stream):
        _ok(lib.flagcxAllReduce(send, recv, count, dtype, op, self.handle, stream), "flagcxAllReduce")

    def reduce(self, send, recv, count, dtype, op, root, stream):
        _ok(lib.flagcxReduce(send, recv, count, dtype, op, root, self.handle, stream), "flagcxReduce")

    def reduce_scatter(self, send, recv, recvcount, dtype, op, stream):
        _ok(lib.flagcxReduceScatter(send, recv, recvcount, dtype, op, self.handle, stream), "flagcxReduceScatter")

    def all_gather(self, send, recv, sendcount, dtype, stream):
        _ok(lib.flagcxAllGather(send, recv, sendcount, dtype, self.handle, stream), "flagcxAllGather")

    def broadcast(self, send, recv, count, dtype, root, stream):
        _ok(lib.flagcxBroadcast(send, recv, count, dtype, root, self.handle, stream), "flagcxBroadcast")

    def send(self, buf, count, dtype, peer, stream):
        _ok(lib.flagcxSend(buf, count, dtype, peer, self.handle, stream), "flagcxSend")

    def recv(self, buf, count, dtype, peer, stream):
        _ok(lib.flagcxRecv(buf, count, dtype, peer, self.handle, stream), "flagcxRecv")

    def barrier(self, stream):
        _ok(lib.flagcxBarrier(self.handle, stream), "flagcxBarrier")

    def group_start(self):
        _ok(lib.flagcxGroupStart(self.handle), "flagcxGroupStart")

    def group_end(self):
        _ok(lib.flagcxGroupEnd(self.handle), "flagcxGroupEnd")


def join(size, id_bytes=None):
    """All ``size`` ranks of one new communicator."""
    uid = id_bytes or new_id()
    return [Rank.from_id(uid, size, r) for r in range(size)]
