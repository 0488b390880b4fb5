"""The reference-named Python binding (flagcx_amd/wrapper.py) driven the way
the reference's own collective tests drive libflagcx: communicators from a
unique id, one call per rank, closed-form expectations
(test/unittest/runner/coll_allreduce.cpp:9-37, coll_reducescatter.cpp,
coll_allgather.cpp, test/unittest/kernel/coll_deviceptr_allreduce.cpp:72-73)."""
import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd.wrapper import FLAGCXLibrary, flagcxDataTypeEnum as DT, flagcxRedOpTypeEnum as OP
from tests.util import DevBufs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fx(dev):
    return FLAGCXLibrary()


def _group(fx, n):
    uid = fx.flagcxGetUniqueId()
    same = fx.unique_id_from_bytes(bytes(bytearray(uid.internal)))     # the id as another process would receive it
    return [fx.flagcxCommInitRank(n, uid if r % 2 else same, r) for r in range(n)]


def test_life_cycle_and_errors(dev, fx):
    assert fx.flagcxGetVersion() == "0.1.0"
    assert fx.flagcxGetErrorString(N.INVALID_ARGUMENT) == "invalid argument"
    comms = _group(fx, 3)
    assert [fx.flagcxCommUserRank(c) for c in comms] == [0, 1, 2] and fx.flagcxCommCount(comms[1]) == 3
    stream = fx.adaptor_stream_create()
    assert fx.flagcxGetErrorString(N.NOT_SUPPORTED) == "not supported"
    with pytest.raises(RuntimeError, match="invalid argument"):
        fx.flagcxAllReduce(1 << 12, 1 << 12, 4, DT.flagcxFloat, OP.flagcxNumOps, comms[0], stream)
    with pytest.raises(RuntimeError, match="invalid argument"):
        fx.flagcxAllReduce(None, None, 4, DT.flagcxFloat, OP.flagcxSum, comms[0], stream)
    with pytest.raises(ValueError):
        fx.unique_id_from_bytes(b"short")
    # a rank joins a communicator once; a late joiner must agree on its size
    uid = fx.flagcxGetUniqueId()
    half = fx.flagcxCommInitRank(2, uid, 0)
    with pytest.raises(RuntimeError, match="invalid argument"):
        fx.flagcxCommInitRank(2, uid, 0)
    with pytest.raises(RuntimeError, match="invalid argument"):
        fx.flagcxCommInitRank(3, uid, 1)
    other = fx.flagcxCommInitRank(2, uid, 1)
    comms += [half, other]
    for c in comms:
        fx.flagcxCommDestroy(c)
    fx.adaptor_stream_destroy(stream)


@pytest.mark.parametrize("n", [2, 8])
def test_reference_closed_forms(dev, fx, n):
    count = 1 << 16
    comms = _group(fx, n)
    stream = fx.adaptor_stream_create()
    raw = dev.raw_stream(stream.value)
    wrapped = fx.adaptor_stream_copy(raw)            # a foreign stream handed over the way a torch stream is
    idx = np.arange(count)
    with DevBufs(dev) as b:
        # allreduce: send[i] = rank*1000 + i%10  ->  n(n-1)/2*1000 + n*(i%10)
        ds = [b.put((r * 1000 + idx % 10).astype(np.float32)) for r in range(n)]
        dr = [b.alloc(count * 4) for _ in range(n)]
        for r in range(n):
            fx.flagcxAllReduce(ds[r], dr[r], count, DT.flagcxFloat, OP.flagcxSum, comms[r], wrapped if r else stream)
        fx.adaptor_stream_synchronize(stream)
        want = (n * (n - 1) // 2 * 1000 + n * (idx % 10)).astype(np.float32)
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[r], count, np.float32), want)
        # device-pointer test's pattern: every element rank+1 -> n(n+1)/2, in place, int64
        di = [b.put(np.full(count, r + 1, np.int64)) for r in range(n)]
        for r in range(n):
            fx.flagcxAllReduce(di[r], di[r], count, DT.flagcxInt64, OP.flagcxSum, comms[r], stream)
        fx.flagcxBarrier(comms[0], stream)
        for r in range(1, n):
            fx.flagcxBarrier(comms[r], stream)
        fx.adaptor_stream_synchronize(stream)
        assert (dev.to_host(di[n - 1], count, np.int64) == n * (n + 1) // 2).all()
        # reduce to root 1, max: rank n-1 wins everywhere
        for r in range(n):
            fx.flagcxReduce(ds[r], dr[r] if r == 1 else None, count, DT.flagcxFloat, OP.flagcxMax, 1, comms[r], stream)
        # reduce-scatter + all-gather == allreduce
        rc = count // n
        drs = [b.alloc(rc * 4) for _ in range(n)]
        dag = [b.alloc(count * 4) for _ in range(n)]
        for r in range(n):
            fx.flagcxReduceScatter(ds[r], drs[r], rc, DT.flagcxFloat, OP.flagcxSum, comms[r], stream)
        for r in range(n):
            fx.flagcxAllGather(drs[r], dag[r], rc, DT.flagcxFloat, comms[r], stream)
        # broadcast rank 0's send buffer; send / recv rank 0 -> rank n-1 inside a group bracket
        dbc = [b.alloc(count * 4) for _ in range(n)]
        for r in range(n):
            fx.flagcxBroadcast(ds[r], dbc[r], count, DT.flagcxFloat, 0, comms[r], stream)
        dp2p = b.alloc(count * 4)
        fx.flagcxGroupStart(comms[0])
        fx.flagcxSend(ds[0], count, DT.flagcxFloat, n - 1, comms[0], stream)
        fx.flagcxRecv(dp2p, count, DT.flagcxFloat, 0, comms[n - 1], stream)
        fx.flagcxGroupEnd(comms[0])
        fx.adaptor_stream_synchronize(stream)
        assert np.array_equal(dev.to_host(dr[1], count, np.float32), ((n - 1) * 1000 + idx % 10).astype(np.float32))
        for r in (0, n - 1):
            assert np.array_equal(dev.to_host(dag[r], count, np.float32), want)
            assert np.array_equal(dev.to_host(dbc[r], count, np.float32), (idx % 10).astype(np.float32))
        assert np.array_equal(dev.to_host(dp2p, count, np.float32), (idx % 10).astype(np.float32))
    for c in comms:
        fx.flagcxCommDestroy(c)
    fx.adaptor_stream_free(wrapped)
    fx.adaptor_stream_destroy(stream)
