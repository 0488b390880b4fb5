"""Python-side callers of the kernel C ABI (pointers are plain integers)."""
import ctypes as C

import numpy as np

from . import _native as N

lib = N.lib


def _ptr_array(ptrs):
    return (C.c_void_p * len(ptrs))(*ptrs)


def reduce_copy(out, ins, count, dtype, op, first=0, stream=None):
    return lib.fx_reduce_copy(out, _ptr_array(ins), len(ins), count, dtype, op, first, stream)


def reduce2(out, a, b, count, dtype, op, stream=None):
    return lib.fx_reduce2(out, a, b, count, dtype, op, stream)


def make_slices(descs):
    """descs: iterable of (ins, out, count)."""
    descs = list(descs)
    arr = (N.SliceDesc * max(len(descs), 1))()
    for d, (ins, out, count) in zip(arr, descs):
        for p, v in enumerate(ins):
            d.in_[p] = v
        d.out = out
        d.count = count
    return arr, len(descs)


def reduce_slices(descs, k, dtype, op, stream=None):
    arr, n = make_slices(descs)
    return lib.fx_reduce_slices(arr, n, k, dtype, op, stream)


def reduce_bcast_slices(descs, k, nout, dtype, op, stream=None):
    """descs: iterable of (ins, outs, count); op = -1 broadcasts in[0] (count in bytes)."""
    descs = list(descs)
    arr = (N.BcastDesc * max(len(descs), 1))()
    for i, (ins, outs, count) in enumerate(descs):
        for p, ptr in enumerate(ins):
            arr[i].inp[p] = ptr
        for o, ptr in enumerate(outs):
            arr[i].out[o] = ptr
        arr[i].count = count
    return lib.fx_reduce_bcast_slices(arr, len(descs), k, nout, dtype, op, stream)


FOLD_CHAIN, FOLD_TREE, FOLD_KEEP_LOCAL = 0, 1, 2   # include/flagcx_amd/fx_kernels.h


def reduce_ordered(descs, k, nout, dtype, op, order, stream=None):
    """descs as for reduce_bcast_slices; the k inputs of every slice are combined in the given
    association (FOLD_TREE: ins[a] = tree rank a; FOLD_KEEP_LOCAL: ins[0] first, then ins[j] (op) res)."""
    descs = list(descs)
    arr = (N.BcastDesc * max(len(descs), 1))()
    for i, (ins, outs, count) in enumerate(descs):
        for p, ptr in enumerate(ins):
            arr[i].inp[p] = ptr
        for o, ptr in enumerate(outs):
            arr[i].out[o] = ptr
        arr[i].count = count
    return lib.fx_reduce_ordered(arr, len(descs), k, nout, dtype, op, order, stream)


def reduce_bcast(outs, ins, count, dtype, op, first=0, stream=None):
    """One segment, up to 64 inputs folded once into up to 64 outputs; op = -1 copies ins[0] (count in bytes)."""
    return lib.fx_reduce_bcast(_ptr_array(outs), len(outs), _ptr_array(ins), len(ins), count, dtype, op, first, stream)


def reduce_chunks(outs, ins, chunks, dtype, op, stream=None):
    """chunks: iterable of (in_off, out_off, count, first, in_sel, out_sel); op = -1 copies (bytes)."""
    chunks = list(chunks)
    arr = (N.Chunk * max(len(chunks), 1))(*[N.Chunk(*c) for c in chunks])
    return lib.fx_reduce_chunks(_ptr_array(outs), len(outs), _ptr_array(ins), len(ins), arr, len(chunks), dtype, op, stream)


def alltoall(recvs, sends, block_bytes, stream=None):
    """Block i of sends[r] becomes block r of recvs[i]; one launch for any number of ranks up to 64."""
    return lib.fx_alltoall(_ptr_array(recvs), _ptr_array(sends), len(sends), block_bytes, stream)


def copy_slices(descs, stream=None):
    """descs: iterable of (src, dst, nbytes)."""
    arr, n = make_slices(([s], d, b) for s, d, b in descs)
    return lib.fx_copy_slices(arr, n, stream)


class Plan:
    def __init__(self, descs, k, dtype, op):
        arr, n = make_slices(descs)
        self.h = C.c_void_p()
        N.check(lib.fx_plan_create(C.byref(self.h), arr, n, k, dtype, op), "fx_plan_create")

    def launch(self, stream=None):
        return lib.fx_plan_launch(self.h, stream)

    def destroy(self):
        if self.h:
            lib.fx_plan_destroy(self.h)
            self.h = C.c_void_p()


def reduce_slices_static(descs, k, dtype, op, stream=None):
    """fx_plan_create + fx_plan_launch without any allocation; op = -1 copies (count in bytes)."""
    arr, n = make_slices(descs)
    return lib.fx_reduce_slices_static(arr, n, k, dtype, op, stream)


def make_trigger(in1, in2, out, count, nthreads, dtype, op, state=N.SUCCESS + 1):
    t = N.ReduceTrigger()
    lib.fx_trigger_set(C.byref(t), in1, in2, out, count, nthreads, dtype, op, state)
    return t


def trigger_fields(t):
    u = [C.c_uint64() for _ in range(5)]
    i = [C.c_int() for _ in range(3)]
    lib.fx_trigger_get(C.byref(t), *[C.byref(x) for x in u], *[C.byref(x) for x in i])
    return dict(in1=u[0].value, in2=u[1].value, out=u[2].value, count=u[3].value, nthreads=u[4].value,
                dtype=i[0].value, op=i[1].value, state=i[2].value)


def reduce_triggers(triggers, stream=None):
    arr = (N.ReduceTrigger * max(len(triggers), 1))(*triggers)
    return lib.fx_reduce_triggers(arr, len(triggers), stream)


def _sz_array(v):
    return (C.c_size_t * max(len(v), 1))(*[int(x) for x in v])


def pack(packed, sendbuff, counts, displs, dtype, stream=None):
    return lib.fx_pack(packed, sendbuff, _sz_array(counts), _sz_array(displs), len(counts), dtype, stream)


def unpack(recvbuff, packed, counts, displs, dtype, stream=None):
    return lib.fx_unpack(recvbuff, packed, _sz_array(counts), _sz_array(displs), len(counts), dtype, stream)


def split(total, parts, idx):
    c, o = C.c_size_t(), C.c_size_t()
    lib.fx_split(total, parts, idx, C.byref(c), C.byref(o))
    return c.value, o.value


def synth(n, dtype, dist, a, b, seed, stream=0, threads=8):
    """Host array of n synthetic elements (16-bit floats as uint16 bit patterns)."""
    np_dt = N.NP_DTYPE[dtype]
    out = np.empty(n, dtype=np_dt)
    N.check(lib.fx_synth_fill(out.ctypes.data, n, dtype, dist, a, b, seed, stream, threads), "fx_synth_fill")
    return out


SYNTH_UNIFORM, SYNTH_NORMAL, SYNTH_UNIFORM_INT = 0, 1, 2
