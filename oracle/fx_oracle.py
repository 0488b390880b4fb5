"""ctypes access to the CPU checker (oracle/fx_oracle.c).  Test infrastructure:
imported only by tests, the smoke check and the benchmark's CPU-baseline leg."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfx_oracle.so")


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "libfx_oracle.so"], stdout=subprocess.DEVNULL)


if not os.path.exists(_SO):
    build()
lib = C.CDLL(_SO)

_vp, _sz, _i = C.c_void_p, C.c_size_t, C.c_int


class RedNode(C.Structure):
    _fields_ = [("step", C.c_int32), ("rank", C.c_int32), ("in1_buf", C.c_int32), ("in2_buf", C.c_int32),
                ("out_buf", C.c_int32), ("slice", C.c_int32), ("in1_off", C.c_uint64), ("in2_off", C.c_uint64),
                ("out_off", C.c_uint64), ("count", C.c_uint64)]


lib.oracle_reduce_copy.restype = _i
lib.oracle_reduce_copy.argtypes = [_vp, C.POINTER(_vp), _i, _sz, _i, _i, _i]
lib.oracle_reduce_copy_elem.restype = _i
lib.oracle_reduce_copy_elem.argtypes = [_vp, C.POINTER(_vp), _i, _sz, _i, _i, _i]
lib.oracle_reduce2.restype = _i
lib.oracle_reduce2.argtypes = [_vp, _vp, _vp, _sz, _i, _i]
lib.oracle_host_ring_passes.restype = _i
lib.oracle_host_ring_passes.argtypes = [_vp, C.POINTER(_vp), _i, _sz, _i, _i]
lib.oracle_split.restype = None
lib.oracle_split.argtypes = [_sz, _sz, _sz, C.POINTER(_sz), C.POINTER(_sz)]
lib.oracle_nredslices.restype = _sz
lib.oracle_nredslices.argtypes = [_sz, _i, _sz, _sz, _sz]
for _n in ("oracle_plan_ring_ar", "oracle_plan_ring_rs"):
    getattr(lib, _n).restype = _sz
    getattr(lib, _n).argtypes = [_sz, _i, _i, _sz, _sz, C.POINTER(RedNode)]
lib.oracle_plan_locred.restype = _sz
lib.oracle_plan_locred.argtypes = [_sz, _i, _i, _sz, C.POINTER(RedNode)]
lib.oracle_ring_allreduce.restype = _i
lib.oracle_ring_allreduce.argtypes = [C.POINTER(_vp), C.POINTER(_vp), _i, _sz, _i, _i]
lib.oracle_tree_reduce.restype = _i
lib.oracle_tree_reduce.argtypes = [_vp, C.POINTER(_vp), _i, _i, _sz, _i, _i]
lib.oracle_tree_steps.restype = _i
lib.oracle_tree_steps.argtypes = [_i, _i]
lib.oracle_pack.restype = None
lib.oracle_pack.argtypes = [_vp, _vp, C.POINTER(_sz), C.POINTER(_sz), _i, _sz]
lib.oracle_unpack.restype = None
lib.oracle_unpack.argtypes = [_vp, _vp, C.POINTER(_sz), C.POINTER(_sz), _i, _sz]
lib.oracle_alltoallv.restype = None
lib.oracle_alltoallv.argtypes = [C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), _i, _sz]
lib.oracle_trigger_encode.restype = None
lib.oracle_trigger_encode.argtypes = [C.POINTER(C.c_uint64)] + [C.c_uint64] * 5 + [_i] * 3
lib.oracle_trigger_decode.restype = None
lib.oracle_trigger_decode.argtypes = [C.POINTER(C.c_uint64)] + [C.POINTER(C.c_uint64)] * 2 + [C.POINTER(_i)] * 3
lib.oracle_bf16_to_f32.restype = C.c_float
lib.oracle_bf16_to_f32.argtypes = [C.c_uint16]
lib.oracle_f32_to_bf16.restype = C.c_uint16
lib.oracle_f32_to_bf16.argtypes = [C.c_float]
lib.oracle_f16_to_f32.restype = C.c_float
lib.oracle_f16_to_f32.argtypes = [C.c_uint16]
lib.oracle_f32_to_f16.restype = C.c_uint16
lib.oracle_f32_to_f16.argtypes = [C.c_float]
lib.oracle_bootstrap_chunks.restype = None
lib.oracle_bootstrap_chunks.argtypes = [_sz, _i, _sz, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
lib.oracle_bootstrap_reduce_scatter.restype = _i
lib.oracle_bootstrap_reduce_scatter.argtypes = [C.POINTER(_vp), C.POINTER(_vp), _i, C.POINTER(C.c_size_t),
                                                C.POINTER(C.c_size_t), _i, _i]
lib.oracle_bootstrap_allreduce.restype = _i
lib.oracle_bootstrap_allreduce.argtypes = [C.POINTER(_vp), C.POINTER(_vp), _i, _sz, _i, _i]
lib.oracle_set_threads.argtypes = [_i]
lib.oracle_dtype_size.restype = _sz
lib.oracle_dtype_size.argtypes = [_i]


def _ptrs(arrays):
    return (_vp * len(arrays))(*[a.ctypes.data for a in arrays])


def reduce_copy(ins, dtype, op, first=0, out=None):
    """ins: list of equal-length contiguous numpy arrays (uint16 for 16-bit floats)."""
    ins = [np.ascontiguousarray(a) for a in ins]
    if out is None:
        out = np.empty_like(ins[0])
    rc = lib.oracle_reduce_copy(out.ctypes.data, _ptrs(ins), len(ins), ins[0].size, dtype, op, first)
    if rc:
        raise ValueError(f"oracle_reduce_copy rc={rc}")
    return out


def reduce_copy_elem(ins, dtype, op, first=0):
    """16-bit types folded in the element type itself (the reference device kernel's arithmetic); uint16 arrays."""
    ins = [np.ascontiguousarray(a) for a in ins]
    out = np.empty_like(ins[0])
    rc = lib.oracle_reduce_copy_elem(out.ctypes.data, _ptrs(ins), len(ins), ins[0].size, dtype, op, first)
    if rc:
        raise ValueError(f"oracle_reduce_copy_elem rc={rc}")
    return out


def reduce2(a, b, dtype, op):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    out = np.empty_like(a)
    rc = lib.oracle_reduce2(out.ctypes.data, a.ctypes.data, b.ctypes.data, a.size, dtype, op)
    if rc:
        raise ValueError(f"oracle_reduce2 rc={rc}")
    return out


def host_ring_passes(ins, dtype, op):
    ins = [np.ascontiguousarray(a) for a in ins]
    acc = np.empty_like(ins[0])
    rc = lib.oracle_host_ring_passes(acc.ctypes.data, _ptrs(ins), len(ins), ins[0].size, dtype, op)
    if rc:
        raise ValueError(f"oracle_host_ring_passes rc={rc}")
    return acc


def split(total, parts, idx):
    c, o = _sz(), _sz()
    lib.oracle_split(total, parts, idx, C.byref(c), C.byref(o))
    return c.value, o.value


def _plan(fn, *args):
    n = fn(*args, None)
    nodes = (RedNode * max(n, 1))()
    fn(*args, nodes)
    return [nodes[i] for i in range(n)]


def plan_ring_ar(count, nranks, rank, nslices, nred):
    return _plan(lib.oracle_plan_ring_ar, count, nranks, rank, nslices, nred)


def plan_ring_rs(recvcount, nranks, rank, nslices, nred):
    return _plan(lib.oracle_plan_ring_rs, recvcount, nranks, rank, nslices, nred)


def plan_locred(count, nranks, rank, nslices):
    return _plan(lib.oracle_plan_locred, count, nranks, rank, nslices)


def ring_allreduce(sends, dtype, op):
    """Returns the per-rank receive buffers of a hop-by-hop ring allreduce."""
    sends = [np.ascontiguousarray(a) for a in sends]
    recvs = [np.zeros_like(a) for a in sends]
    rc = lib.oracle_ring_allreduce(_ptrs(recvs), _ptrs(sends), len(sends), sends[0].size, dtype, op)
    if rc:
        raise ValueError(f"oracle_ring_allreduce rc={rc}")
    return recvs


def bootstrap_chunks(size, nranks, ts):
    off = (C.c_size_t * nranks)()
    ln = (C.c_size_t * nranks)()
    lib.oracle_bootstrap_chunks(size, nranks, ts, off, ln)
    return list(off), list(ln)


def bootstrap_allreduce(sends, dtype, op):
    """The reference's host ring all-reduce played hop by hop; returns every rank's result."""
    recvs = [np.empty_like(s) for s in sends]
    rc = lib.oracle_bootstrap_allreduce(_ptrs(recvs), _ptrs(sends), len(sends), sends[0].size, dtype, op)
    if rc:
        raise ValueError(f"oracle_bootstrap_allreduce rc={rc}")
    return recvs


def tree_reduce(sends, root, dtype, op):
    """Result at `root` of the reference's binomial-tree reduce."""
    sends = [np.ascontiguousarray(a) for a in sends]
    out = np.empty_like(sends[0])
    rc = lib.oracle_tree_reduce(out.ctypes.data, _ptrs(sends), len(sends), root, sends[0].size, dtype, op)
    if rc:
        raise ValueError(f"oracle_tree_reduce rc={rc}")
    return out


def _szs(v):
    return (_sz * max(len(v), 1))(*[int(x) for x in v])


def pack(send, counts, displs):
    send = np.ascontiguousarray(send)
    out = np.zeros(int(sum(counts)), dtype=send.dtype)
    lib.oracle_pack(out.ctypes.data, send.ctypes.data, _szs(counts), _szs(displs), len(counts), send.itemsize)
    return out


def unpack(recv, packed, counts, displs):
    packed = np.ascontiguousarray(packed)
    lib.oracle_unpack(recv.ctypes.data, packed.ctypes.data, _szs(counts), _szs(displs), len(counts), packed.itemsize)
    return recv


def trigger_encode(in1, in2, out, count, nthreads, dtype, op, state):
    v = (C.c_uint64 * 4)()
    lib.oracle_trigger_encode(v, in1, in2, out, count, nthreads, dtype, op, state)
    return list(v)
