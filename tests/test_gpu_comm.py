"""Communicators joined rank by rank from a unique id (flagcx_amd/comm.py over
the FlagCX-named C entry points), driven the way the reference's own collective
tests drive libflagcx: one call per rank, closed-form expectations
(test/unittest/runner/coll_allreduce.cpp:9-37, coll_reducescatter.cpp,
coll_allgather.cpp, test/unittest/kernel/coll_deviceptr_allreduce.cpp:72-73)."""
import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import comm
from tests.util import DevBufs

pytestmark = pytest.mark.gpu


def _group(n):
    """Even ranks join with the id as another process would receive it (a copy of the bytes)."""
    uid = comm.new_id()
    return [comm.Rank.from_id(uid if r % 2 else bytes(bytearray(uid)), n, r) for r in range(n)]


def _fails_with(code, fn, *args):
    with pytest.raises(N.FlagcxError) as e:
        fn(*args)
    assert e.value.code == code, e.value


def test_life_cycle_and_errors(dev):
    assert comm.version() == (0, 1, 0)
    assert comm.error_text(N.INVALID_ARGUMENT) == "invalid argument"
    assert comm.error_text(N.NOT_SUPPORTED) == "not supported"
    ranks = _group(3)
    assert [r.reported() for r in ranks] == [(0, 3), (1, 3), (2, 3)]
    stream = dev.stream_create()
    _fails_with(N.INVALID_ARGUMENT, ranks[0].all_reduce, 1 << 12, 1 << 12, 4, N.DT_FP32, 5, stream)     # op out of range
    _fails_with(N.INVALID_ARGUMENT, ranks[0].all_reduce, None, None, 4, N.DT_FP32, N.OP_SUM, stream)
    with pytest.raises(ValueError):
        comm.Rank.from_id(b"short", 2, 0)
    # a rank joins a communicator once; a late joiner must agree on its size
    uid = comm.new_id()
    half = comm.Rank.from_id(uid, 2, 0)
    _fails_with(N.INVALID_ARGUMENT, comm.Rank.from_id, uid, 2, 0)
    _fails_with(N.INVALID_ARGUMENT, comm.Rank.from_id, uid, 3, 1)
    other = comm.Rank.from_id(uid, 2, 1)
    for r in ranks + [half, other]:
        r.close()
    dev.stream_destroy(stream)


def test_torch_names_map_without_torch():
    class FakeOp:                                   # what str() / .name of a torch ReduceOp member look like
        def __init__(self, name):
            self.name = name
    assert comm.dtype_code("torch.bfloat16") == N.DT_BF16 and comm.dtype_code("torch.int64") == N.DT_INT64
    assert comm.op_code(FakeOp("PRODUCT")) == N.OP_PROD and comm.op_code("RedOpType.AVG") == N.OP_AVG
    with pytest.raises(TypeError):
        comm.dtype_code("torch.complex64")
    with pytest.raises(TypeError):
        comm.op_code("RedOpType.BAND")


@pytest.mark.parametrize("n", [2, 8])
def test_reference_closed_forms(dev, n):
    count = 1 << 16
    ranks = _group(n)
    stream = dev.stream_create()
    borrowed = comm.borrow_stream(dev.raw_stream(stream), dev.t)   # a foreign stream handed over the way a torch stream is
    idx = np.arange(count)
    with DevBufs(dev) as b:
        # allreduce: send[i] = rank*1000 + i%10  ->  n(n-1)/2*1000 + n*(i%10)
        ds = [b.put((r * 1000 + idx % 10).astype(np.float32)) for r in range(n)]
        dr = [b.alloc(count * 4) for _ in range(n)]
        for r in ranks:
            r.all_reduce(ds[r.index], dr[r.index], count, N.DT_FP32, N.OP_SUM, borrowed if r.index else stream)
        dev.stream_sync(stream)
        want = (n * (n - 1) // 2 * 1000 + n * (idx % 10)).astype(np.float32)
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[r], count, np.float32), want)
        # device-pointer test's pattern: every element rank+1 -> n(n+1)/2, in place, int64
        di = [b.put(np.full(count, r + 1, np.int64)) for r in range(n)]
        for r in ranks:
            r.all_reduce(di[r.index], di[r.index], count, N.DT_INT64, N.OP_SUM, stream)
        for r in ranks:
            r.barrier(stream)
        dev.stream_sync(stream)
        assert (dev.to_host(di[n - 1], count, np.int64) == n * (n + 1) // 2).all()
        # reduce to root 1, max: rank n-1 wins everywhere
        for r in ranks:
            r.reduce(ds[r.index], dr[r.index] if r.index == 1 else None, count, N.DT_FP32, N.OP_MAX, 1, stream)
        # reduce-scatter + all-gather == allreduce
        rc = count // n
        drs = [b.alloc(rc * 4) for _ in range(n)]
        dag = [b.alloc(count * 4) for _ in range(n)]
        for r in ranks:
            r.reduce_scatter(ds[r.index], drs[r.index], rc, N.DT_FP32, N.OP_SUM, stream)
        for r in ranks:
            r.all_gather(drs[r.index], dag[r.index], rc, N.DT_FP32, stream)
        # broadcast rank 0's send buffer; send / recv rank 0 -> rank n-1 inside a group bracket
        dbc = [b.alloc(count * 4) for _ in range(n)]
        for r in ranks:
            r.broadcast(ds[r.index], dbc[r.index], count, N.DT_FP32, 0, stream)
        dp2p = b.alloc(count * 4)
        ranks[0].group_start()
        ranks[0].send(ds[0], count, N.DT_FP32, n - 1, stream)
        ranks[n - 1].recv(dp2p, count, N.DT_FP32, 0, stream)
        ranks[0].group_end()
        dev.stream_sync(stream)
        assert np.array_equal(dev.to_host(dr[1], count, np.float32), ((n - 1) * 1000 + idx % 10).astype(np.float32))
        for r in (0, n - 1):
            assert np.array_equal(dev.to_host(dag[r], count, np.float32), want)
            assert np.array_equal(dev.to_host(dbc[r], count, np.float32), (idx % 10).astype(np.float32))
        assert np.array_equal(dev.to_host(dp2p, count, np.float32), (idx % 10).astype(np.float32))
    for r in ranks:
        r.close()
    comm.return_stream(borrowed, dev.t)
    dev.stream_destroy(stream)


def test_application_flow_through_the_device_handle_and_housekeeping_calls():
    """The calls of a program written against flagcx.h, in the order its perf
    tests make them (test/perf_common.cc:27-110): device handle, unique id,
    communicators, stream, flagcxMemAlloc + flagcxCommRegister buffers, an
    all-reduce with a closed form, deregistration, finalize, destroy / abort."""
    import ctypes as C
    L = N.lib
    handler = C.c_void_p()
    N.check(L.flagcxHandleInit(C.byref(handler)), "flagcxHandleInit")
    uid_p, comm_p, dev_p = C.cast(handler, C.POINTER(C.c_void_p))[0:3]
    assert uid_p is None and comm_p is None and dev_p, "a zeroed group with its device handle filled in"
    ops = C.cast(dev_p, C.POINTER(C.c_void_p))
    assert all(ops[i] for i in range(28)), "every device operation is there"
    RES = C.c_int
    fn = lambda i, *argtypes: C.CFUNCTYPE(RES, *argtypes)(ops[i])      # index = position in flagcx.h:143-185
    device_sync, device_memcpy = fn(0), fn(1, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p)
    set_device, get_count = fn(5, C.c_int), fn(7, C.POINTER(C.c_int))
    stream_create, stream_destroy, stream_sync = fn(10, C.POINTER(C.c_void_p)), fn(11, C.c_void_p), fn(14, C.c_void_p)
    ngpu = C.c_int()
    N.check(get_count(C.byref(ngpu)), "getDeviceCount")
    assert ngpu.value >= 1
    N.check(set_device(0), "setDevice")
    stream = C.c_void_p()
    N.check(stream_create(C.byref(stream)), "streamCreate")

    n, count = 3, 100003
    uid = C.create_string_buffer(256)
    N.check(L.flagcxGetUniqueId(uid), "flagcxGetUniqueId")
    comms = [C.c_void_p() for _ in range(n)]
    for r in range(n):
        N.check(L.flagcxCommInitRank(C.byref(comms[r]), n, uid, r), "flagcxCommInitRank")
    send, recv, hs, hr = ([C.c_void_p() for _ in range(n)] for _ in range(4))
    idx = np.arange(count)
    for r in range(n):
        N.check(L.flagcxMemAlloc(C.byref(send[r]), count * 4, 0), "flagcxMemAlloc")
        N.check(L.flagcxMemAlloc(C.byref(recv[r]), count * 4, 0), "flagcxMemAlloc")
        N.check(L.flagcxCommRegister(comms[r], send[r], count * 4, C.byref(hs[r]), 0), "flagcxCommRegister")
        N.check(L.flagcxCommRegister(comms[r], recv[r], count * 4, C.byref(hr[r]), 0), "flagcxCommRegister")
        assert hs[r].value == send[r].value
        host = (r * 1000 + idx % 10).astype(np.float32)              # coll_allreduce.cpp:9-37
        N.check(device_memcpy(send[r], host.ctypes.data, count * 4, N.MEMCPY_H2D, None), "deviceMemcpy")
    for r in range(n):
        N.check(L.flagcxAllReduce(send[r], recv[r], count, N.DT_FP32, N.OP_SUM, comms[r], stream), "flagcxAllReduce")
    N.check(stream_sync(stream), "streamSynchronize")
    want = (n * (n - 1) // 2 * 1000 + n * (idx % 10)).astype(np.float32)
    for r in range(n):
        got = np.empty(count, np.float32)
        N.check(device_memcpy(got.ctypes.data, recv[r], count * 4, N.MEMCPY_D2H, None), "deviceMemcpy")
        assert np.array_equal(got, want)

    v, err = C.c_int(-1), C.c_int(-1)
    N.check(L.flagcxIsHomoComm(comms[0], C.byref(v)), "flagcxIsHomoComm")
    assert v.value == 1
    N.check(L.flagcxCommGetDeviceNumber(comms[1], C.byref(v)), "flagcxCommGetDeviceNumber")
    assert v.value == 0
    N.check(L.flagcxCommGetAsyncError(comms[2], C.byref(err)), "flagcxCommGetAsyncError")
    assert err.value == N.SUCCESS and L.flagcxGetLastError(comms[0]) == b""
    assert L.flagcxCommSuspend(comms[0]) == N.INVALID_USAGE and L.flagcxCommResume(comms[0]) == N.INVALID_USAGE
    win = C.c_void_p(1)
    assert L.flagcxCommWindowRegister(comms[0], send[0], count * 4, C.byref(win), 1, 0) == N.NOT_SUPPORTED and not win.value
    for r in range(n):
        N.check(L.flagcxCommDeregister(comms[r], hs[r], 0), "flagcxCommDeregister")
        N.check(L.flagcxCommDeregister(comms[r], hr[r], 0), "flagcxCommDeregister")
        N.check(L.flagcxCommFinalize(comms[r]), "flagcxCommFinalize")
    N.check(L.flagcxCommAbort(comms[0]), "flagcxCommAbort")
    for r in range(1, n):
        N.check(L.flagcxCommDestroy(comms[r]), "flagcxCommDestroy")
    for r in range(n):
        N.check(L.flagcxMemFree(send[r], 0), "flagcxMemFree")
        N.check(L.flagcxMemFree(recv[r], 0), "flagcxMemFree")
    N.check(device_sync(), "deviceSynchronize")
    N.check(stream_destroy(stream), "streamDestroy")
    N.check(L.flagcxHandleFree(handler), "flagcxHandleFree")
