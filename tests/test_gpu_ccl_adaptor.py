"""The CCL-adaptor plugin driven through its function table, as FlagCX's homo
runner drives a vendor CCL (flagcx/runner/homo_runner.cc:8-22): communicators
created rank by rank from one unique id, then the collectives of the
reference's runner tests (test/unittest/runner/coll_*.cpp) with their closed
forms."""
import ctypes as C

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import ccl_adaptor
from oracle import fx_oracle as O
from tests.util import DevBufs, seeded_inputs

pytestmark = pytest.mark.gpu
OK = N.SUCCESS


@pytest.fixture(scope="module")
def ccl():
    return ccl_adaptor.load_plugin()


@pytest.fixture()
def stream(dev):
    s = dev.stream_create()
    yield s
    dev.stream_destroy(s)


def make_comms(ccl, n):
    uid = C.c_void_p()
    assert ccl.getUniqueId(C.byref(uid)) == OK and uid.value
    comms = []
    for r in range(n):
        c = C.c_void_p()
        assert ccl.commInitRank(C.byref(c), n, uid, r, None) == OK and c.value
        comms.append(c.value)
    return comms, uid


def destroy(ccl, comms):
    for c in comms:
        assert ccl.commDestroy(c) == OK


def test_communicator_queries_and_memory(dev, ccl):
    v = C.c_int()
    assert ccl.getVersion(C.byref(v)) == OK and v.value > 0
    assert ccl.getErrorString(N.INVALID_ARGUMENT) == b"invalid argument"
    comms, uid = make_comms(ccl, 4)
    uid2 = C.c_void_p()
    assert ccl.getUniqueId(C.byref(uid2)) == OK
    assert C.string_at(uid.value, 24) != C.string_at(uid2.value, 24)        # ids differ
    for r, c in enumerate(comms):
        cnt, rank, devno, err = C.c_int(), C.c_int(), C.c_int(-1), C.c_int(-1)
        assert ccl.commCount(c, C.byref(cnt)) == OK and cnt.value == 4
        assert ccl.commUserRank(c, C.byref(rank)) == OK and rank.value == r
        assert ccl.commGetDeviceNumber(c, C.byref(devno)) == OK and devno.value == 0
        assert ccl.commGetAsyncError(c, C.byref(err)) == OK and err.value == OK
        assert ccl.getLastError(c) == b""
    # a rank that does not fit the group
    bad = C.c_void_p()
    assert ccl.commInitRank(C.byref(bad), 4, uid2, 4, None) == N.INVALID_ARGUMENT
    # staged buffers are cached per direction and grow on demand
    b1, b2, b3 = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert ccl.getStagedBuffer(comms[0], C.byref(b1), 1 << 20, 0) == OK and b1.value
    assert ccl.getStagedBuffer(comms[0], C.byref(b2), 1 << 16, 0) == OK and b2.value == b1.value
    assert ccl.getStagedBuffer(comms[0], C.byref(b3), 1 << 20, 1) == OK and b3.value not in (None, b1.value)
    p, h = C.c_void_p(), C.c_void_p()
    assert ccl.memAlloc(C.byref(p), 4096) == OK and p.value
    assert ccl.commRegister(comms[1], p, 4096, C.byref(h)) == OK and h.value
    assert ccl.commDeregister(comms[1], h) == OK
    assert ccl.memFree(p) == OK
    assert ccl.commWindowRegister(comms[0], None, 0, None, 0) == N.NOT_SUPPORTED
    assert ccl.commResume(comms[0]) == N.INVALID_USAGE and ccl.commSuspend(comms[0]) == N.INVALID_USAGE
    assert ccl.groupStart() == OK and ccl.groupEnd() == OK
    assert ccl.commFinalize(comms[0]) == OK
    destroy(ccl, comms)


def test_reducing_collectives_closed_forms(dev, ccl, stream):
    n, count = 8, 1 << 20                         # 4 MiB float buffers as runner/main_mpi.cpp:33-80
    comms, _ = make_comms(ccl, n)
    i = np.arange(count)
    sends = [(r * 1000 + i % 10).astype(np.float32) for r in range(n)]
    with DevBufs(dev) as b:
        ds = [b.put(a) for a in sends]
        dr = [b.alloc(count * 4) for _ in range(n)]
        # coll_allreduce.cpp:9-37
        for r in range(n):
            assert ccl.allReduce(ds[r], dr[r], count, N.DT_FP32, N.OP_SUM, comms[r], stream) == OK
        dev.stream_sync(stream)
        want = (n * (n - 1) // 2 * 1000 + n * (i % 10)).astype(np.float32)
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[r], count, np.float32), want)
        # coll_reduce.cpp: same data, root 0
        dev.memset(dr[0], 0, count * 4)
        for r in range(n):
            assert ccl.reduce(ds[r], dr[r], count, N.DT_FP32, N.OP_SUM, 0, comms[r], stream) == OK
        dev.stream_sync(stream)
        assert np.array_equal(dev.to_host(dr[0], count, np.float32), want)
        # coll_reducescatter.cpp:27-39 style: block r of the sum lands on rank r
        rc = count // n
        for r in range(n):
            assert ccl.reduceScatter(ds[r], dr[r], rc, N.DT_FP32, N.OP_SUM, comms[r], stream) == OK
        dev.stream_sync(stream)
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[r], rc, np.float32), want[r * rc:(r + 1) * rc])
        # seeded bf16 data against the oracle
        bf = seeded_inputs(N.DT_BF16, n, 300001, seed=5)
        dbs = [b.put(a) for a in bf]
        for r in range(n):
            assert ccl.allReduce(dbs[r], dr[r], 300001, N.DT_BF16, N.OP_SUM, comms[r], stream) == OK
        dev.stream_sync(stream)
        wantb = O.reduce_copy(bf, N.DT_BF16, N.OP_SUM)
        for r in (0, 7):
            assert np.array_equal(dev.to_host(dr[r], 300001, np.uint16), wantb)
        assert ccl.allReduce(ds[0], dr[0], count, N.DT_FP32, 5, comms[0], stream) == N.INVALID_ARGUMENT
        for r in range(n):      # avg, the op the torch backend maps ReduceOp.AVG to (backend_flagcx.cpp:21-25)
            assert ccl.allReduce(ds[r], dr[r], count, N.DT_FP32, N.OP_AVG, comms[r], stream) == OK
        dev.stream_sync(stream)
        assert np.array_equal(dev.to_host(dr[n - 1], count, np.float32), O.reduce_copy(sends, N.DT_FP32, N.OP_AVG))
    destroy(ccl, comms)


@pytest.mark.parametrize("n", [2, 8])
def test_legacy_suite_identical_inputs(dev, ccl, stream, n):
    """The reference's first collective suite (test/unittest/main.cpp:15-310): every
    rank sends the pattern i % 10 as fp32 and the result, divided by the number of
    ranks where it is a sum, is the pattern again.  The pattern's first 1000 values
    are the data file that suite ships (test/unittest/baseline_result.txt, kept
    here as tests/golden/reference_baseline_result.txt)."""
    import os
    fixture = np.loadtxt(os.path.join(os.path.dirname(__file__), "golden", "reference_baseline_result.txt"),
                         dtype=np.float32)
    count = 1000 * n
    i = np.arange(count)
    pattern = (i % 10).astype(np.float32)
    assert fixture.shape == (1000,) and np.array_equal(pattern[:1000], fixture)
    comms, _ = make_comms(ccl, n)
    call = lambda f, *a: [f(*[x[r] if isinstance(x, list) else x for x in a], comms[r], stream) for r in range(n)]
    with DevBufs(dev) as b:
        ds = [b.put(pattern) for _ in range(n)]
        dr = [b.alloc(count * 4) for _ in range(n)]
        get = lambda r, cnt=count: dev.to_host(dr[r], cnt, np.float32)
        assert set(call(ccl.allReduce, ds, dr, count, N.DT_FP32, N.OP_SUM)) == {OK}          # :15-58
        dev.stream_sync(stream)
        for r in range(n):
            assert np.array_equal(get(r) / n, pattern) and np.array_equal((get(r) / n)[:1000], fixture)
        assert set(call(ccl.allReduce, ds, dr, count, N.DT_FP32, N.OP_AVG)) == {OK}          # the division done by the op
        dev.stream_sync(stream)
        assert np.array_equal(get(n - 1)[:1000], fixture)
        sc = count // n
        assert set(call(ccl.allGather, ds, dr, sc, N.DT_FP32)) == {OK}                       # :60-102
        dev.stream_sync(stream)
        for r in range(n):                               # sc is a multiple of 10, so the gathered blocks continue the pattern
            assert np.array_equal(get(r), pattern)
        assert set(call(ccl.reduceScatter, ds, dr, sc, N.DT_FP32, N.OP_SUM)) == {OK}         # :104-146
        dev.stream_sync(stream)
        for r in range(n):
            assert np.array_equal(get(r, sc) / n, pattern[r * sc:(r + 1) * sc])
        dev.memset(dr[0], 0, count * 4)
        assert set(call(ccl.reduce, ds, dr, count, N.DT_FP32, N.OP_SUM, 0)) == {OK}          # :148-190
        dev.stream_sync(stream)
        assert np.array_equal(get(0) / n, pattern)
        dev.memset(dr[0], 0, count * 4)
        assert set(call(ccl.gather, ds, dr, sc, N.DT_FP32, 0)) == {OK}                       # :192-234
        dev.stream_sync(stream)
        assert np.array_equal(get(0), pattern)
        dev.upload(ds[0], i.astype(np.float32))                                              # :236-277: root sends 0, 1, 2, ...
        assert set(call(ccl.scatter, ds, dr, sc, N.DT_FP32, 0)) == {OK}
        dev.stream_sync(stream)
        for r in range(n):
            assert np.array_equal(get(r, sc), i[r * sc:(r + 1) * sc].astype(np.float32))
        dev.upload(ds[0], pattern)
        assert set(call(ccl.broadcast, ds, dr, count, N.DT_FP32, 0)) == {OK}                 # :279-310
        dev.stream_sync(stream)
        for r in range(n):
            assert np.array_equal(get(r), pattern)
    destroy(ccl, comms)


def test_byte_moving_collectives(dev, ccl, stream):
    n, count = 4, 70001
    comms, _ = make_comms(ccl, n)
    rng = np.random.default_rng(2)
    blocks = [rng.integers(0, 2**32, n * count, dtype=np.uint64).astype(np.uint32) for _ in range(n)]
    with DevBufs(dev) as b:
        ds = [b.put(a) for a in blocks]
        dr = [b.alloc(n * count * 4) for _ in range(n)]
        call = lambda f, *a: [f(*[x[r] if isinstance(x, list) else x for x in a], comms[r], stream) for r in range(n)]
        # allGather (coll_allgather.cpp): block r of every recvbuff is rank r's first `count` elements
        assert set(call(ccl.allGather, ds, dr, count, N.DT_FP32)) == {OK}
        dev.stream_sync(stream)
        want = np.concatenate([a[:count] for a in blocks])
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[r], n * count, np.uint32), want)
        # broadcast (coll_broadcast.cpp:9-35 uses root 0; here root 2)
        assert set(call(ccl.broadcast, ds, dr, count, N.DT_FP32, 2)) == {OK}
        dev.stream_sync(stream)
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[r], count, np.uint32), blocks[2][:count])
        # gather (coll_gather.cpp:10-37: chunk r on the root is rank r's data) to root 1; scatter (coll_scatter.cpp:12-38) from root 3
        assert set(call(ccl.gather, ds, dr, count, N.DT_FP32, 1)) == {OK}
        dev.stream_sync(stream)
        assert np.array_equal(dev.to_host(dr[1], n * count, np.uint32), want)
        assert set(call(ccl.scatter, ds, dr, count, N.DT_FP32, 3)) == {OK}
        dev.stream_sync(stream)
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[r], count, np.uint32), blocks[3][r * count:(r + 1) * count])
        # alltoall (coll_alltoall.cpp): block i of rank r -> block r of rank i; then in place
        assert set(call(ccl.alltoAll, ds, dr, count, N.DT_FP32)) == {OK}
        dev.stream_sync(stream)
        for i in range(n):
            want_i = np.concatenate([blocks[r][i * count:(i + 1) * count] for r in range(n)])
            assert np.array_equal(dev.to_host(dr[i], n * count, np.uint32), want_i)
        assert set(call(ccl.alltoAll, ds, ds, count, N.DT_FP32)) == {OK}
        dev.stream_sync(stream)
        for i in range(n):
            want_i = np.concatenate([blocks[r][i * count:(i + 1) * count] for r in range(n)])
            assert np.array_equal(dev.to_host(ds[i], n * count, np.uint32), want_i)
    destroy(ccl, comms)


def test_send_recv_pairs(dev, ccl, stream):
    n, count = 3, 12345
    comms, _ = make_comms(ccl, n)
    data = seeded_inputs(N.DT_FP32, n, count, seed=9)
    s2 = dev.stream_create()
    with DevBufs(dev) as b:
        ds = [b.put(a) for a in data]
        dr = [b.alloc(count * 4) for _ in range(n)]
        # ring shift as coll_sendrecv.cpp:12-31: rank r sends to r+1; receives posted first for one pair, sends first for the others
        assert ccl.recv(dr[1], count, N.DT_FP32, 0, comms[1], s2) == OK
        for r in range(n):
            assert ccl.send(ds[r], count, N.DT_FP32, (r + 1) % n, comms[r], stream) == OK
        assert ccl.recv(dr[2], count, N.DT_FP32, 1, comms[2], stream) == OK
        assert ccl.recv(dr[0], count, N.DT_FP32, 2, comms[0], s2) == OK
        dev.stream_sync(stream)
        dev.stream_sync(s2)
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[(r + 1) % n], count, np.float32), data[r])
        # size mismatch is reported to the later caller
        assert ccl.send(ds[0], 10, N.DT_FP32, 1, comms[0], stream) == OK
        assert ccl.recv(dr[1], 11, N.DT_FP32, 0, comms[1], stream) == N.INVALID_ARGUMENT
        assert ccl.send(ds[0], 10, N.DT_FP32, 5, comms[0], stream) == N.INVALID_ARGUMENT     # no such peer
        dev.stream_sync(stream)
    dev.stream_destroy(s2)
    destroy(ccl, comms)
