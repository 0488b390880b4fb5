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
