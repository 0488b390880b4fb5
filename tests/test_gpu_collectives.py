"""Collective-shaped entry points over simulated ranks: closed forms of the
reference's own collective tests, parity with the hop-by-hop ring oracle, and
the custom allreduce hook."""
import ctypes as C

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import sim as S
from oracle import fx_oracle as O
from tests.util import DTYPES, DevBufs, assert_parity, is_nan16, seeded_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture()
def stream(dev):
    s = dev.stream_create()
    yield s
    dev.stream_destroy(s)


def _allreduce(dev, stream, sends, dtype, op, inplace=False, **cfg):
    n, count = len(sends), sends[0].size
    es = N.DTYPE_SIZE[dtype]
    with DevBufs(dev) as b, S.SimGroup(n, **cfg) as g:
        ds = [b.put(a) for a in sends]
        dr = ds if inplace else [b.alloc(count * es) for _ in range(n)]
        N.check(g.all_reduce(ds, dr, count, dtype, op, stream), "flagcxAllReduce")
        dev.stream_sync(stream)
        return [dev.to_host(p, count, N.NP_DTYPE[dtype]) for p in dr]


@pytest.mark.parametrize("n", [1, 2, 3, 8])
@pytest.mark.parametrize("algo", [S.ALGO_DIRECT, S.ALGO_RING])
def test_allreduce_closed_forms(dev, stream, n, algo):
    count = 4 * 1024 * 1024 // 4 if n == 8 else 10007       # runner/main_mpi.cpp:33-80 uses 4 MiB float buffers
    i = np.arange(count)
    # coll_allreduce.cpp:9-37
    sends = [(r * 1000 + i % 10).astype(np.float32) for r in range(n)]
    want = (n * (n - 1) // 2 * 1000 + n * (i % 10)).astype(np.float32)
    for got in _allreduce(dev, stream, sends, N.DT_FP32, N.OP_SUM, algo=algo):
        assert np.array_equal(got, want)
    # coll_deviceptr_allreduce.cpp:72-73
    sends = [np.full(count, r + 1, np.float32) for r in range(n)]
    for got in _allreduce(dev, stream, sends, N.DT_FP32, N.OP_SUM, algo=algo, inplace=True):
        assert (got == n * (n + 1) / 2).all()
    # test/perf/host_api/test_allreduce.cpp:20-32 (exact in fp32)
    sends = [((i % 10) * 2.0 ** (r % 30)).astype(np.float32) for r in range(n)]
    want = sum(s.astype(np.float64) for s in sends).astype(np.float32)
    for got in _allreduce(dev, stream, sends, N.DT_FP32, N.OP_SUM, algo=algo, nslices=3):
        assert np.array_equal(got, want)


@pytest.mark.parametrize("dname", ["fp32", "int32", "fp64", "int64", "uint8"])
@pytest.mark.parametrize("n,count,nslices,nred", [(8, 100003, 8, 2), (5, 77, 2, 0), (4, 3, 1, 0), (2, 65536, 4, 3)])
def test_allreduce_matches_ring_oracle_bit_for_bit(dev, stream, dname, n, count, nslices, nred):
    """fp32 sums depend on order: the ring algorithm and the direct k-way
    algorithm in ring order must both reproduce the hop-by-hop oracle."""
    dtype = DTYPES[dname]
    sends = seeded_inputs(dtype, n, count, seed=13)
    for op in (N.OP_SUM, N.OP_PROD, N.OP_MAX, N.OP_MIN):
        want = O.ring_allreduce(sends, dtype, op)
        for cfg in (dict(algo=S.ALGO_RING), dict(algo=S.ALGO_DIRECT, order=S.ORDER_RING)):
            for inplace in (False, True):
                got = _allreduce(dev, stream, sends, dtype, op, inplace=inplace, nslices=nslices, nredslices=nred,
                                 redslicesize=1024, **cfg)
                for r in range(n):
                    assert_parity(got[r], want[r], dtype, op, f"{cfg} inplace={inplace} rank {r} op={op}")


@pytest.mark.parametrize("dname", ["bf16", "fp16"])
def test_allreduce_16bit_rank_order(dev, stream, dname):
    """Default order = rank order = the custom allreduce's peer loop; 16-bit sums
    accumulate in fp32 across all 8 ranks and round once."""
    dtype = DTYPES[dname]
    n, count = 8, 262144 + 5
    sends = seeded_inputs(dtype, n, count, seed=1)
    for op in (N.OP_SUM, N.OP_MAX):
        want = O.reduce_copy(sends, dtype, op)
        for got in _allreduce(dev, stream, sends, dtype, op, nslices=8, nredslices=2):
            assert_parity(got, want, dtype, op, f"allreduce {dname} op={op}")


def test_reduce_reducescatter_allgather(dev, stream):
    n, rc = 8, 5001
    dtype, es = N.DT_FP32, 4
    sends = seeded_inputs(dtype, n, n * rc, seed=3)
    with DevBufs(dev) as b, S.SimGroup(n) as g:
        ds = [b.put(a) for a in sends]
        # Reduce to root 3; recvbuff NULL elsewhere (flagcx.h:365-366)
        droot = b.alloc(n * rc * es)
        recvs = [droot if r == 3 else None for r in range(n)]
        N.check(g.reduce(ds, recvs, n * rc, dtype, N.OP_SUM, 3, stream))
        dev.stream_sync(stream)
        assert_parity(dev.to_host(droot, n * rc, np.float32), O.reduce_copy(sends, dtype, N.OP_SUM), dtype, N.OP_SUM)
        # ReduceScatter: rank r gets block r; ring order and ring algorithm agree bit for bit
        for cfg in (dict(algo=S.ALGO_RING, nslices=2, nredslices=3), dict(algo=S.ALGO_DIRECT, order=S.ORDER_RING),
                    dict(algo=S.ALGO_DIRECT, order=S.ORDER_RANK)):
            g.configure(**cfg)
            dr = [b.alloc(rc * es) for _ in range(n)]
            N.check(g.reduce_scatter(ds, dr, rc, dtype, N.OP_SUM, stream))
            dev.stream_sync(stream)
            for r in range(n):
                first = (r + 1) % n if cfg.get("order", S.ORDER_RING) == S.ORDER_RING else 0
                want = O.reduce_copy([s[r * rc:(r + 1) * rc] for s in sends], dtype, N.OP_SUM, first=first)
                assert_parity(dev.to_host(dr[r], rc, np.float32), want, dtype, N.OP_SUM, f"RS {cfg} rank {r}")
        # closed form of coll_reducescatter.cpp:27-39 style data
        # AllGather: block r of every recvbuff is rank r's sendbuff; in place when send == recv + r*count
        g.configure(algo=S.ALGO_DIRECT, order=S.ORDER_RANK, nslices=1, nredslices=0)
        dg = [b.alloc(n * rc * es) for _ in range(n)]
        small = [s[:rc] for s in sends]
        for r in range(n):
            dev.upload(dg[r] + r * rc * es, small[r])
        N.check(g.all_gather([dg[r] + r * rc * es for r in range(n)], dg, rc, dtype, stream))
        dev.stream_sync(stream)
        want = np.concatenate(small)
        for r in range(n):
            assert np.array_equal(dev.to_host(dg[r], n * rc, np.float32), want)


@pytest.mark.parametrize("dname", ["fp32", "bf16"])
@pytest.mark.parametrize("n", [2, 3, 5, 6, 8, 11])
def test_reduce_in_tree_order_matches_the_reference_tree(dev, stream, n, dname):
    """flagcxReduce through the reference's uniRunner is a binomial tree
    (uni_runner_impl.cc:1266-1557); sums must match it bit for bit when that
    order is asked for, for every root, in place and out of place -- fp32, and
    bf16 where every step of the tree rounds to the element type.  Up to eight
    ranks run as one launch, eleven as one launch per round."""
    count = 70003
    dtype = DTYPES[dname]
    es, npdt = N.DTYPE_SIZE[dtype], N.NP_DTYPE[dtype]
    bits = np.uint32 if es == 4 else np.uint16
    sends = seeded_inputs(dtype, n, count, seed=n)
    for root in sorted({0, 1 % n, n - 1}):
        for op in (N.OP_SUM, N.OP_PROD):
            want = O.tree_reduce(sends, root, dtype, op)
            with DevBufs(dev) as b, S.SimGroup(n, order=2) as g:      # FX_ORDER_TREE
                ds = [b.put(a) for a in sends]
                dout = b.alloc(count * es)
                N.check(g.reduce(ds, [dout if r == root else None for r in range(n)], count, dtype, op, root, stream))
                dev.stream_sync(stream)
                assert np.array_equal(dev.to_host(dout, count, npdt).view(bits), want.view(bits)), f"tree n={n} root={root}"
                N.check(g.reduce(ds, [ds[r] if r == root else None for r in range(n)], count, dtype, op, root, stream))
                dev.stream_sync(stream)
                assert np.array_equal(dev.to_host(ds[root], count, npdt).view(bits), want.view(bits)), "tree in place"
    if n > 3 and dname == "fp32":   # and it is a different association from the rank-order fold
        a = O.tree_reduce(sends, 0, N.DT_FP32, N.OP_SUM)
        assert not np.array_equal(a.view(np.uint32), O.reduce_copy(sends, N.DT_FP32, N.OP_SUM).view(np.uint32))


def test_reduce_scatter_in_place(dev, stream):
    n, rc = 4, 3003
    sends = seeded_inputs(N.DT_INT32, n, n * rc, seed=8)
    for cfg in (dict(algo=S.ALGO_RING), dict(algo=S.ALGO_DIRECT)):
        with DevBufs(dev) as b, S.SimGroup(n, order=S.ORDER_RING, **cfg) as g:
            ds = [b.put(a) for a in sends]
            dr = [ds[r] + r * rc * 4 for r in range(n)]           # flagcx.h:439
            N.check(g.reduce_scatter(ds, dr, rc, N.DT_INT32, N.OP_SUM, stream))
            dev.stream_sync(stream)
            for r in range(n):
                want = O.reduce_copy([s[r * rc:(r + 1) * rc] for s in sends], N.DT_INT32, N.OP_SUM)
                assert np.array_equal(dev.to_host(dr[r], rc, np.int32), want)


def test_alltoallv_matches_oracle(dev, stream):
    n = 8
    rng = np.random.default_rng(3)
    counts = np.exp(rng.uniform(0, np.log(50000), (n, n))).astype(np.int64)     # counts[r][i]: r -> i
    counts[2, 5] = 0
    counts[4, 4] = 0
    sd = np.zeros((n, n), np.int64)
    rd = np.zeros((n, n), np.int64)
    slen, rlen = [], []
    for r in range(n):
        order, pos = rng.permutation(n), 0
        for i in order:
            pos += int(rng.integers(0, 5))
            sd[r, i] = pos
            pos += int(counts[r, i])
        slen.append(pos + 3)
        order, pos = rng.permutation(n), 0
        for i in order:
            pos += int(rng.integers(0, 5))
            rd[r, i] = pos
            pos += int(counts[i, r])
        rlen.append(pos + 3)
    sends = [rng.integers(0, 2**32, slen[r], dtype=np.uint64).astype(np.uint32) for r in range(n)]
    want = [np.zeros(rlen[r], np.uint32) for r in range(n)]
    szs = lambda a: (C.c_size_t * a.size)(*[int(x) for x in a.ravel()])
    vp = lambda arrs: (C.c_void_p * n)(*[a.ctypes.data for a in arrs])
    O.lib.oracle_alltoallv(vp(want), vp(sends), szs(counts), szs(sd), szs(rd), n, 4)
    with DevBufs(dev) as b, S.SimGroup(n) as g:
        ds = [b.put(a) for a in sends]
        dr = [b.alloc(rlen[r] * 4) for r in range(n)]
        for r in range(n):
            dev.memset(dr[r], 0, rlen[r] * 4)
        N.check(g.all_to_allv(ds, counts, sd, dr, counts.T, rd, N.DT_FP32, stream))
        dev.stream_sync(stream)
        for r in range(n):
            assert np.array_equal(dev.to_host(dr[r], rlen[r], np.uint32), want[r]), r
        bad = counts.T.copy()
        bad[0, 1] += 1                                             # receiver expects more than is sent
        assert g.all_to_allv(ds, counts, sd, dr, bad, rd, N.DT_FP32, stream) == N.INVALID_ARGUMENT
        # a rank with something to send and no send buffer is refused before anything is launched
        assert g.all_to_allv([None] + ds[1:], counts, sd, dr, counts.T, rd, N.DT_FP32, stream) == N.INVALID_ARGUMENT
        # in place (send == recv, uneven blocks laid out back to back): goes through the staging slots
        blk = np.array([[1000 + 37 * ((r + i) % n) for i in range(n)] for r in range(n)], np.int64)   # symmetric
        disp = np.concatenate([np.zeros((n, 1), np.int64), np.cumsum(blk, axis=1)[:, :-1]], axis=1)
        bufs = [rng.integers(0, 2**32, int(blk[r].sum()), dtype=np.uint64).astype(np.uint32) for r in range(n)]
        dbuf = [b.put(a) for a in bufs]
        N.check(g.all_to_allv(dbuf, blk, disp, dbuf, blk.T, disp, N.DT_FP32, stream))
        dev.stream_sync(stream)
        for i in range(n):
            got = dev.to_host(dbuf[i], bufs[i].size, np.uint32)
            for r in range(n):
                src = bufs[r][disp[r, i]:disp[r, i] + blk[r, i]]
                assert np.array_equal(got[disp[i, r]:disp[i, r] + blk[r, i]], src), (i, r)


def test_custom_allreduce_hook(dev, stream):
    n, count = 8, (8 << 20) // 2            # the reference's 8 MiB staged window, bf16
    dtype = N.DT_BF16
    sends = seeded_inputs(dtype, n, count, seed=1)
    with DevBufs(dev) as b, S.SimGroup(n) as g:
        ds = [b.put(a) for a in sends]
        dr = [b.alloc(count * 2) for _ in range(n)]
        # no windows registered -> caller falls through (flagcx.cc:2673-2680)
        assert g.custom_all_reduce(ds, dr, count, dtype, N.OP_SUM, stream) == N.NOT_SUPPORTED
        wins = [b.alloc(8 << 20) for _ in range(n)]
        N.check(g.register_windows(wins, 8 << 20))
        assert g.custom_all_reduce(ds, dr, count + 1, dtype, N.OP_SUM, stream) == N.NOT_SUPPORTED   # > window
        assert g.custom_all_reduce(ds, dr, count, dtype, 5, stream) == N.NOT_SUPPORTED               # the hook only declines
        for op in (N.OP_SUM, N.OP_MIN, N.OP_AVG):
            N.check(g.custom_all_reduce(ds, dr, count, dtype, op, stream))
            dev.stream_sync(stream)
            want = O.reduce_copy(sends, dtype, op)
            for r in range(n):
                assert_parity(dev.to_host(dr[r], count, np.uint16), want, dtype, op, f"custom AR rank {r}")
        # odd count (the reference drops the tail, custom_allreduce.cu:383-384) and in-place on the window
        for r in range(n):
            dev.upload(wins[r], sends[r][:1001])
        N.check(g.custom_all_reduce(wins, dr, 1001, dtype, N.OP_SUM, stream))
        dev.stream_sync(stream)
        want = O.reduce_copy([s[:1001] for s in sends], dtype, N.OP_SUM)
        assert_parity(dev.to_host(dr[5], 1001, np.uint16), want, dtype, N.OP_SUM, "odd count")


@pytest.mark.parametrize("n", [2, 4, 8])
def test_custom_allreduce_reference_intranode_cases(dev, stream, n):
    """The reference's own checks of its intra-node all-reduce kernel, run through
    the hook on registered windows: every rank contributes rank + 1, the result is
    n (n + 1) / 2 everywhere -- in place on the registered buffer
    (test/unittest/device_api/test_device_api_intra.cpp:363-389, tolerance 1e-1
    there) and out of place into a receive buffer
    (test/perf/device_api/test_allreduce_intranode.cpp:196-211, tolerance 1e-3);
    exact here.  Then the fixture pattern (i % 10) + seed of
    test/fixtures/test_utils.hpp:28-34 with seed = rank, compared the way its
    verifyBuffer does (relative 1e-5, :11-26) and exactly."""
    count = 1 << 20                                     # 4 MiB of fp32, inside the 8 MiB window
    with DevBufs(dev) as b, S.SimGroup(n) as g:
        wins = [b.alloc(8 << 20) for _ in range(n)]
        N.check(g.register_windows(wins, 8 << 20))
        dr = [b.alloc(count * 4) for _ in range(n)]
        for r in range(n):
            dev.upload(wins[r], np.full(count, r + 1, np.float32))
        N.check(g.custom_all_reduce(wins, dr, count, N.DT_FP32, N.OP_SUM, stream))      # out of place
        N.check(g.custom_all_reduce(wins, wins, count, N.DT_FP32, N.OP_SUM, stream))    # in place on the windows
        dev.stream_sync(stream)
        for r in range(n):
            assert (dev.to_host(dr[r], count, np.float32) == n * (n + 1) / 2).all()
            assert (dev.to_host(wins[r], count, np.float32) == n * (n + 1) / 2).all()
        i = np.arange(count)
        for r in range(n):
            dev.upload(wins[r], ((i % 10) + r).astype(np.float32))
        N.check(g.custom_all_reduce(wins, dr, count, N.DT_FP32, N.OP_SUM, stream))
        dev.stream_sync(stream)
        want = (n * (i % 10) + n * (n - 1) // 2).astype(np.float32)
        for r in range(n):
            got = dev.to_host(dr[r], count, np.float32)
            rel = np.abs(got.astype(np.float64) - want) / np.maximum(np.abs(want.astype(np.float64)), 1e-10)
            assert rel.max() <= 1e-5 and np.array_equal(got, want)


def test_group_misuse_is_reported(dev, stream):
    with DevBufs(dev) as b, S.SimGroup(2) as g:
        p = b.alloc(64)
        lib = N.lib
        assert lib.flagcxAllReduce(p, p, 4, N.DT_FP32, N.OP_SUM, g.comms[0], stream) == N.SUCCESS
        assert lib.flagcxAllReduce(p, p, 4, N.DT_FP32, N.OP_SUM, g.comms[0], stream) == N.INVALID_USAGE   # rank 0 twice
        assert lib.flagcxAllReduce(p, p, 4, N.DT_FP32, N.OP_SUM, g.comms[0], stream) == N.SUCCESS
        assert lib.flagcxAllReduce(p, p, 8, N.DT_FP32, N.OP_SUM, g.comms[1], stream) == N.INVALID_ARGUMENT  # count differs
        assert lib.flagcxReduce(p, p, 4, N.DT_FP32, N.OP_SUM, 2, g.comms[0], stream) == N.INVALID_ARGUMENT   # bad root
        assert lib.flagcxAllReduce(p, p, 4, N.DT_FP32, N.OP_SUM, g.comms[0], None) == N.INVALID_ARGUMENT     # no stream
        cnt, rank = C.c_int(), C.c_int()
        assert lib.flagcxCommCount(g.comms[1], C.byref(cnt)) == N.SUCCESS and cnt.value == 2
        assert lib.flagcxCommUserRank(g.comms[1], C.byref(rank)) == N.SUCCESS and rank.value == 1
        dev.stream_sync(stream)


def test_ranks_on_different_streams(dev):
    """Each simulated rank posts on its own stream; the last post waits for the
    others' pending uploads and the others wait for the result."""
    n, count = 4, 1 << 20
    sends = seeded_inputs(N.DT_FP32, n, count, seed=17)
    streams = [dev.stream_create() for _ in range(n)]
    try:
        with DevBufs(dev) as b, S.SimGroup(n) as g:
            ds = [b.alloc(count * 4) for _ in range(n)]
            dr = [b.alloc(count * 4) for _ in range(n)]
            hosts = [dev.malloc(count * 4, N.MEM_HOST) for _ in range(n)]
            for r in range(n):
                C.memmove(hosts[r], sends[r].ctypes.data, count * 4)
                N.check(dev.t.deviceMemcpy(ds[r], hosts[r], count * 4, N.MEMCPY_H2D, streams[r], None))  # async, own stream
            N.check(g.all_reduce(ds, dr, count, N.DT_FP32, N.OP_SUM, streams))
            out = [np.empty(count, np.float32) for _ in range(n)]
            for r in range(n):          # read back on each rank's OWN stream, no device-wide sync
                N.check(dev.t.deviceMemcpy(hosts[r], dr[r], count * 4, N.MEMCPY_D2H, streams[r], None))
                dev.stream_sync(streams[r])
                C.memmove(out[r].ctypes.data, hosts[r], count * 4)
            want = O.reduce_copy(sends, N.DT_FP32, N.OP_SUM)
            for r in range(n):
                assert np.array_equal(out[r], want)
            for h in hosts:
                dev.free(h, N.MEM_HOST)
    finally:
        for s in streams:
            dev.stream_destroy(s)


def test_one_host_thread_per_rank(dev):
    """FlagCX applications drive each rank from its own thread on its own stream.
    Eight threads post 30 all-reduces each (alternating op), never synchronising
    with one another on the host; every result must equal the oracle's."""
    import threading
    n, count, rounds = 8, 100003, 30
    sends = seeded_inputs(N.DT_FP32, n, count, seed=21)
    want = {op: O.reduce_copy(sends, N.DT_FP32, op) for op in (N.OP_SUM, N.OP_MAX)}
    errors = []
    with DevBufs(dev) as b, S.SimGroup(n) as g:
        ds = [b.put(a) for a in sends]
        dr = [[b.alloc(count * 4) for _ in range(n)] for _ in range(2)]
        streams = [dev.stream_create() for _ in range(n)]

        def rank_main(r):
            try:
                dev.set_device()
                for it in range(rounds):
                    op = (N.OP_SUM, N.OP_MAX)[it % 2]
                    # a collective is matched by arrival order, so a rank may only post round it
                    # once every rank has posted round it-1: the barrier models the application's own
                    # per-step structure and involves no device synchronisation
                    gate.wait()
                    rc = N.lib.flagcxAllReduce(ds[r], dr[it % 2][r], count, N.DT_FP32, op, g.comms[r], streams[r])
                    if rc != N.SUCCESS:
                        errors.append((r, it, rc))
                dev.stream_sync(streams[r])
            except Exception as e:                      # noqa: BLE001 - reported below
                errors.append((r, repr(e)))
                gate.abort()

        gate = threading.Barrier(n)
        threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=60)
        assert not errors, errors
        assert not any(t.is_alive() for t in threads)
        for r in range(n):
            assert_parity(dev.to_host(dr[1][r], count, np.float32), want[N.OP_MAX], N.DT_FP32, N.OP_MAX, f"rank {r}")
            assert_parity(dev.to_host(dr[0][r], count, np.float32), want[N.OP_SUM], N.DT_FP32, N.OP_SUM, f"rank {r}")
        for s in streams:
            dev.stream_destroy(s)


def test_rendezvous_mode_orders_later_work_after_the_collective(dev):
    """One host thread per rank, each on its own stream, written the way the
    reference's per-process tests are (coll_allreduce.cpp:9-37): upload, all-reduce,
    download on the same stream right after the call, synchronise, check -- with
    no host barrier between ranks.  Only a call that returns after the collective
    is enqueued makes the download see the result."""
    import threading
    n, count, rounds = 8, 50001, 12
    idx = np.arange(count)
    errors = []
    with DevBufs(dev) as b, S.SimGroup(n, sync=S.SYNC_RENDEZVOUS) as g:
        dbuf = [b.alloc(count * 4) for _ in range(n)]
        dtmp = [b.alloc(count * 4) for _ in range(n)]

        def rank_main(r):
            try:
                dev.set_device()
                s = dev.stream_create()
                host = np.empty(count, np.float32)
                for it in range(rounds):
                    src = ((r + it) * 1000 + idx % 10).astype(np.float32)      # kept alive until the stream is drained
                    dev.upload(dbuf[r], src, s)
                    N.check(N.lib.flagcxAllReduce(dbuf[r], dbuf[r], count, N.DT_FP32, N.OP_SUM, g.comms[r], s))
                    dev.download(host, dbuf[r], s)
                    dev.stream_sync(s)
                    want = (sum(q + it for q in range(n)) * 1000 + n * (idx % 10)).astype(np.float32)
                    if not np.array_equal(host, want):
                        errors.append((r, it, "allreduce", host[:4].tolist(), want[:4].tolist()))
                    # ring shift: send own block to the right neighbour, receive from the left one
                    src = np.full(count, r * 100 + it, np.float32)
                    dev.upload(dbuf[r], src, s)
                    if r % 2 == 0:      # even ranks send first, odd ranks receive first: no cyclic wait
                        N.check(N.lib.flagcxSend(dbuf[r], count, N.DT_FP32, (r + 1) % n, g.comms[r], s))
                        N.check(N.lib.flagcxRecv(dtmp[r], count, N.DT_FP32, (r - 1) % n, g.comms[r], s))
                    else:
                        N.check(N.lib.flagcxRecv(dtmp[r], count, N.DT_FP32, (r - 1) % n, g.comms[r], s))
                        N.check(N.lib.flagcxSend(dbuf[r], count, N.DT_FP32, (r + 1) % n, g.comms[r], s))
                    dev.download(host, dtmp[r], s)
                    dev.stream_sync(s)
                    if not (host == ((r - 1) % n) * 100 + it).all():
                        errors.append((r, it, "sendrecv", host[:4].tolist()))
                    N.check(N.lib.flagcxBarrier(g.comms[r], s))     # nobody overwrites dbuf while a neighbour reads it
                    dev.stream_sync(s)
                dev.stream_destroy(s)
            except Exception as e:                      # noqa: BLE001 - reported below
                errors.append((r, repr(e)))

        threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
        assert not any(t.is_alive() for t in threads)
        assert not errors, errors[:4]


def test_rendezvous_ring_exchange_inside_a_group_bracket(dev, monkeypatch):
    """The usual thread-per-rank pattern: every rank runs GroupStart, Send(next),
    Recv(prev), GroupEnd -- all of them send FIRST.  Outside a bracket that would
    leave every thread asleep in its send; inside one the posts are remembered
    and the bracket's end waits for the partners.  It must finish by itself, well
    inside the rendezvous time-out (set long enough here that a pass through the
    time-out path would show in the elapsed time), with the right data."""
    import threading
    import time
    monkeypatch.setenv("FX_SIM_RENDEZVOUS_TIMEOUT_MS", "15000")
    n, count, rounds = 8, 40003, 10
    errors = []
    with DevBufs(dev) as b, S.SimGroup(n, sync=S.SYNC_RENDEZVOUS) as g:
        dsend = [b.alloc(count * 4) for _ in range(n)]
        drecv = [b.alloc(count * 4) for _ in range(n)]

        def rank_main(r):
            try:
                dev.set_device()
                s = dev.stream_create()
                host = np.empty(count, np.float32)
                for it in range(rounds):
                    src = np.full(count, r * 100 + it, np.float32)
                    dev.upload(dsend[r], src, s)
                    N.check(N.lib.flagcxGroupStart(g.comms[r]))
                    N.check(N.lib.flagcxSend(dsend[r], count, N.DT_FP32, (r + 1) % n, g.comms[r], s))
                    N.check(N.lib.flagcxRecv(drecv[r], count, N.DT_FP32, (r - 1) % n, g.comms[r], s))
                    N.check(N.lib.flagcxGroupEnd(g.comms[r]))
                    dev.download(host, drecv[r], s)
                    dev.stream_sync(s)
                    if not (host == ((r - 1) % n) * 100 + it).all():
                        errors.append((r, it, host[:4].tolist()))
                    N.check(N.lib.flagcxBarrier(g.comms[r], s))     # nobody overwrites dsend while a neighbour reads it
                    dev.stream_sync(s)
                dev.stream_destroy(s)
            except Exception as e:                      # noqa: BLE001 - reported below
                errors.append((r, repr(e)))

        t0 = time.time()
        threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
        assert not any(t.is_alive() for t in threads)
        assert not errors, errors[:4]
        assert time.time() - t0 < 12, "the exchange went through the time-out path"
    assert N.lib.flagcxGroupEnd(None) == N.INVALID_USAGE            # no bracket open on this thread


def test_rendezvous_bracket_with_two_streams_per_rank(dev, monkeypatch):
    """One bracket whose two halves sit on two streams of the same rank, both busy:
    each pending half carries a mark of its own, so the partner of the first half
    waits for THAT stream's earlier work, not for wherever the rank's last mark
    went.  Every rank sends on stream A data that a long-running fill on A writes
    just before, and receives on stream B."""
    import threading
    monkeypatch.setenv("FX_SIM_RENDEZVOUS_TIMEOUT_MS", "15000")
    n, count, rounds = 4, 2_000_003, 6
    errors = []
    with DevBufs(dev) as b, S.SimGroup(n, sync=S.SYNC_RENDEZVOUS) as g:
        dsend = [b.alloc(count * 4) for _ in range(n)]
        drecv = [b.alloc(count * 4) for _ in range(n)]
        busy = [b.alloc(64 << 20) for _ in range(n)]

        def rank_main(r):
            try:
                dev.set_device()
                sa, sb = dev.stream_create(), dev.stream_create()
                host = np.empty(count, np.float32)
                for it in range(rounds):
                    src = np.full(count, r * 100 + it, np.float32)
                    dev.memset(busy[r], it, 64 << 20, sa)          # keeps stream A busy ahead of the upload
                    dev.upload(dsend[r], src, sa)
                    dev.memset(busy[r], it + 1, 64 << 20, sb)      # and stream B busy too, so both halves get marks
                    N.check(N.lib.flagcxGroupStart(g.comms[r]))
                    N.check(N.lib.flagcxSend(dsend[r], count, N.DT_FP32, (r + 1) % n, g.comms[r], sa))
                    N.check(N.lib.flagcxRecv(drecv[r], count, N.DT_FP32, (r - 1) % n, g.comms[r], sb))
                    N.check(N.lib.flagcxGroupEnd(g.comms[r]))
                    dev.download(host, drecv[r], sb)
                    dev.stream_sync(sb)
                    dev.stream_sync(sa)
                    if not (host == ((r - 1) % n) * 100 + it).all():
                        errors.append((r, it, host[:4].tolist(), host[-2:].tolist()))
                    N.check(N.lib.flagcxBarrier(g.comms[r], sa))
                    dev.stream_sync(sa)
                dev.stream_destroy(sa)
                dev.stream_destroy(sb)
            except Exception as e:                      # noqa: BLE001 - reported below
                errors.append((r, repr(e)))

        threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
        assert not any(t.is_alive() for t in threads)
        assert not errors, errors[:4]


def test_alltoall_stages_whenever_a_send_buffer_meets_a_receive_buffer(dev, stream):
    """Not only a rank in place: rank 0 receives into what rank 1 sends, and rank 2's
    receive buffer overlaps rank 0's send buffer partly.  The one-launch kernel reads
    and writes concurrently, so such calls must go through staging; the result is
    what the original send contents say."""
    n, blk = 3, 50_001
    rng = np.random.default_rng(12)
    sends = [rng.integers(-1000, 1000, n * blk, dtype=np.int32) for _ in range(n)]
    with DevBufs(dev) as b, S.SimGroup(n) as g:
        arena = b.alloc(4 * n * blk * 4 + 4096)
        ds = [arena, arena + n * blk * 4, arena + 2 * n * blk * 4]
        own = b.alloc(n * blk * 4)
        dr = [ds[1],                      # rank 0 receives into rank 1's send buffer
              own,
              ds[0] + 1000 * 4]           # rank 2's receive buffer overlaps rank 0's send buffer (and runs into rank 1's)
        for d, a in zip(ds, sends):
            dev.upload(d, a)
        for r in range(n):
            N.check(N.lib.flagcxAlltoAll(ds[r], dr[r], blk, N.DT_INT32, g.comms[r], stream))
        dev.stream_sync(stream)
        # rank 1's own buffer is touched by nobody else: it must hold block 1 of every rank's ORIGINAL send data
        want1 = np.concatenate([sends[r][blk:2 * blk] for r in range(n)])
        assert np.array_equal(dev.to_host(own, n * blk, np.int32), want1)
        # rank 0 and rank 2 overlap each other's results where dr[2] runs into ds[1] = dr[0]; what lies outside that
        # overlap is checked: the first part of rank 2's buffer (inside ds[0]) and the tail of rank 0's
        want2 = np.concatenate([sends[r][2 * blk:3 * blk] for r in range(n)])
        got2 = dev.to_host(dr[2], n * blk, np.int32)
        free2 = n * blk - 1000            # elements of dr[2] that lie before ds[1] starts
        assert np.array_equal(got2[:free2], want2[:free2])


def test_rendezvous_times_out_when_a_rank_never_arrives(dev, stream, monkeypatch):
    import threading
    monkeypatch.setenv("FX_SIM_RENDEZVOUS_TIMEOUT_MS", "200")
    n = 4
    codes = {}
    with DevBufs(dev) as b, S.SimGroup(n, sync=S.SYNC_RENDEZVOUS) as g:
        p = b.alloc(1024)

        def rank_main(r):
            codes[r] = N.lib.flagcxAllReduce(p, p, 16, N.DT_FP32, N.OP_SUM, g.comms[r], stream)

        threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(n - 1)]    # rank 3 stays away
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=20)
        assert codes == {0: N.INTERNAL_ERROR, 1: N.INTERNAL_ERROR, 2: N.INTERNAL_ERROR}
        # nothing was enqueued and the group is usable again
        g.configure(sync=S.SYNC_GROUP)
        N.check(g.all_reduce([p] * n, [p] * n, 0, N.DT_FP32, N.OP_SUM, stream))
        dev.stream_sync(stream)


@pytest.mark.parametrize("dname", ["fp32", "fp64", "int32", "uint8"])
@pytest.mark.parametrize("n,count", [(8, 100003), (3, 10), (4, 2), (5, 77777), (12, 40001)])
def test_host_order_matches_the_reference_host_ring(dev, stream, dname, n, count):
    """FX_ORDER_HOST: the chunks and the fold of the reference's host path
    (bootstrap.cc:787-942), bit for bit, for all-reduce, reduce and
    reduce-scatter, in place and out of place; +-0 ties of max / min included."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    npdt = N.NP_DTYPE[dtype]
    sends = seeded_inputs(dtype, n, count, seed=n + count)
    if dname in ("fp32", "fp64"):                     # widen the exponent range so that association shows
        rng = np.random.default_rng(count)
        sends = [(a * 10.0 ** rng.integers(-3, 9, count)).astype(npdt) for a in sends]
        for r, a in enumerate(sends):                 # and plant zeros of both signs for the tie rule
            a[:min(count, 8)] = [(0.0, -0.0)[(r + i) % 2] for i in range(min(count, 8))]
        for i in range(8, min(count, 8 + 3 * n)):     # one NaN per position, on a rank that moves along the ring:
            sends[i % n][i] = np.nan                  # which operands survive it depends on where it enters the chain
    for op in (N.OP_SUM, N.OP_MAX, N.OP_MIN):
        want = O.bootstrap_allreduce(sends, dtype, op)[0]
        for inplace in (False, True):
            got = _allreduce(dev, stream, sends, dtype, op, inplace=inplace, order=3)
            for r in range(n):
                assert_parity(got[r], want, dtype, op, f"host order allreduce n={n} rank {r} op={op}")
        with DevBufs(dev) as b, S.SimGroup(n, order=3) as g:
            ds = [b.put(a) for a in sends]
            root = n - 1
            dout = b.alloc(count * es)
            N.check(g.reduce(ds, [dout if r == root else None for r in range(n)], count, dtype, op, root, stream))
            dev.stream_sync(stream)
            assert_parity(dev.to_host(dout, count, npdt), want, dtype, op, f"host order reduce n={n}")
    # reduce-scatter: chunk r = elements [r * rc, (r + 1) * rc) ends on rank r, same chain
    rc = max(count // n, 1)
    part = [a[:n * rc] if a.size >= n * rc else np.resize(a, n * rc) for a in sends]
    off = (C.c_size_t * n)(*[r * rc * es for r in range(n)])
    ln = (C.c_size_t * n)(*[rc * es] * n)
    outs = [np.empty(rc, npdt) for _ in range(n)]
    vp = lambda arrs: (C.c_void_p * n)(*[a.ctypes.data for a in arrs])
    for op in (N.OP_SUM, N.OP_MIN):
        assert O.lib.oracle_bootstrap_reduce_scatter(vp(outs), vp(part), n, off, ln, dtype, op) == 0
        with DevBufs(dev) as b, S.SimGroup(n, order=3) as g:
            ds = [b.put(a) for a in part]
            dr = [b.alloc(rc * es) for _ in range(n)]
            N.check(g.reduce_scatter(ds, dr, rc, dtype, op, stream))
            dev.stream_sync(stream)
            for r in range(n):
                assert_parity(dev.to_host(dr[r], rc, npdt), outs[r], dtype, op, f"host order reduce-scatter rank {r}")


@pytest.mark.parametrize("dname", ["bf16", "fp16"])
def test_host_order_max_min_of_16_bit_floats_with_nan(dev, stream, dname):
    """max / min select an input's bits, so the host ring's step-by-step result is
    defined for the 16-bit types too (their sums are not comparable: the ring would
    round at every hop).  NaNs enter the chain at every position."""
    dtype, n, count = DTYPES[dname], 5, 30011
    sends = seeded_inputs(dtype, n, count, seed=17)
    nan = 0x7fc0 if dname == "bf16" else 0x7e00
    for i in range(4 * n):
        sends[i % n][i] = nan
        sends[(i + 2) % n][i + 100] = nan ^ 0x8000          # negative NaN, two ranks further on
    for op in (N.OP_MAX, N.OP_MIN):
        want = O.bootstrap_allreduce(sends, dtype, op)[0]
        for inplace in (False, True):
            got = _allreduce(dev, stream, sends, dtype, op, inplace=inplace, order=3)
            for r in range(n):
                assert np.array_equal(got[r], want), f"{dname} op={op} rank {r} inplace={inplace}"


def test_single_rank_and_empty_collectives(dev, stream):
    """nranks == 1 is a copy when out of place and nothing when in place
    (uni_runner_impl.cc:359-379, bootstrap.cc:1001-1006); count == 0 is accepted
    everywhere and touches nothing."""
    count = 1000
    x = np.arange(count, dtype=np.float32)
    with DevBufs(dev) as b, S.SimGroup(1) as g:
        dx, dy = b.put(x), b.alloc(count * 4)
        for order in (S.ORDER_RANK, S.ORDER_RING, S.ORDER_TREE, S.ORDER_HOST):
            for algo in (S.ALGO_DIRECT, S.ALGO_RING):
                g.configure(order=order, algo=algo)
                dev.memset(dy, 0, count * 4)
                N.check(g.all_reduce([dx], [dy], count, N.DT_FP32, N.OP_SUM, stream))
                N.check(g.all_reduce([dx], [dx], count, N.DT_FP32, N.OP_MAX, stream))       # in place
                dev.stream_sync(stream)
                assert np.array_equal(dev.to_host(dy, count, np.float32), x)
                assert np.array_equal(dev.to_host(dx, count, np.float32), x)
        for call in (lambda: g.reduce([dx], [dy], count, N.DT_FP32, N.OP_AVG, 0, stream),
                     lambda: g.reduce_scatter([dx], [dy], count, N.DT_FP32, N.OP_SUM, stream),
                     lambda: g.all_gather([dx], [dy], count, N.DT_FP32, stream)):
            dev.memset(dy, 0, count * 4)
            N.check(call())
            dev.stream_sync(stream)
            assert np.array_equal(dev.to_host(dy, count, np.float32), x)
    with DevBufs(dev) as b, S.SimGroup(4) as g:
        p = [b.alloc(64) for _ in range(4)]
        for q in p:
            dev.memset(q, 0x77, 64)
        zeros = np.zeros((4, 4), np.int64)
        for order in (S.ORDER_RANK, S.ORDER_HOST):
            g.configure(order=order)
            N.check(g.all_reduce(p, p, 0, N.DT_FP32, N.OP_SUM, stream))
            N.check(g.reduce(p, p, 0, N.DT_BF16, N.OP_MAX, 2, stream))
            N.check(g.reduce_scatter(p, p, 0, N.DT_INT8, N.OP_PROD, stream))
        N.check(g.all_gather(p, p, 0, N.DT_FP64, stream))
        N.check(g.all_to_allv(p, zeros, zeros, p, zeros, zeros, N.DT_FP32, stream))
        dev.stream_sync(stream)
        for q in p:
            assert (dev.to_host(q, 64, np.uint8) == 0x77).all()
        # arguments the API must refuse without touching the device
        assert g.reduce(p, p, 4, N.DT_FP32, N.OP_SUM, 4, stream) == N.INVALID_ARGUMENT          # root out of range
        assert N.lib.flagcxAllReduce(p[0], p[0], 4, N.DT_FP32, N.OP_SUM, g.comms[0], None) == N.INVALID_ARGUMENT
        assert N.lib.flagcxAllReduce(None, p[0], 4, N.DT_FP32, N.OP_SUM, g.comms[0], stream) == N.INVALID_ARGUMENT


@pytest.mark.parametrize("dname", ["fp32", "fp64", "int32", "uint8", "int64"])
@pytest.mark.parametrize("n,count", [(8, 100003), (3, 10), (4, 2), (5, 77777), (2, 1 << 20)])
def test_host_staged_allreduce_matches_host_order_and_oracle(dev, stream, dname, n, count):
    """fxHostStagedAllReduce is the reference's CPU path end to end
    (host_runner.cc:236-289 over bootstrap.cc:787-942): device to host through
    the device adaptor's deviceMemcpy, ring all-reduce with the host loops, host
    to device.  Its result must be the hop-by-hop oracle's and, bit for bit, what
    the device computes under FX_ORDER_HOST; its timers must add up."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    npdt = N.NP_DTYPE[dtype]
    sends = seeded_inputs(dtype, n, count, seed=3 * n + count)
    if dname in ("fp32", "fp64"):
        rng = np.random.default_rng(count)
        sends = [(a * 10.0 ** rng.integers(-3, 9, count)).astype(npdt) for a in sends]
        for r, a in enumerate(sends):
            a[:min(count, 8)] = [(0.0, -0.0)[(r + i) % 2] for i in range(min(count, 8))]
        for i in range(8, min(count, 8 + 3 * n)):
            sends[i % n][i] = np.nan
    with DevBufs(dev) as b, S.HostStaged(n, dev.t.deviceMemcpy) as hs, S.SimGroup(n, order=S.ORDER_HOST) as g:
        ds = [b.put(a) for a in sends]
        dr = [b.alloc(count * es) for _ in range(n)]
        ddev = [b.alloc(count * es) for _ in range(n)]
        for op in (N.OP_SUM, N.OP_MAX, N.OP_MIN):
            want = O.bootstrap_allreduce(sends, dtype, op)
            rc, timers = hs.all_reduce(ds, dr, count, dtype, op)
            N.check(rc, "fxHostStagedAllReduce")
            N.check(g.all_reduce(ds, ddev, count, dtype, op, stream))
            dev.stream_sync(stream)
            for r in range(n):
                got = dev.to_host(dr[r], count, npdt)
                assert np.array_equal(got.view(np.uint8), want[r].view(np.uint8)), f"rank {r} op {op} vs the oracle"
                on_device = dev.to_host(ddev[r], count, npdt)
                assert np.array_equal(got.view(np.uint8), on_device.view(np.uint8)), f"rank {r} op {op} vs FX_ORDER_HOST"
                t = timers[r]
                # (the ring's own buffer allocation is counted in both `alloc` and `comm`, as in the reference)
                assert t["total"] >= t["mem_d2h"] + t["comm"] + t["mem_h2d"] and t["comm"] >= t["calc"] + t["mem"]
                assert t["mem_d2h"] > 0 and t["mem_h2d"] > 0 and (n == 1 or count < n or t["calc"] > 0)
        # in place on the device buffers
        rc, _ = hs.all_reduce(ds, ds, count, dtype, N.OP_SUM)
        N.check(rc)
        want = O.bootstrap_allreduce(sends, dtype, N.OP_SUM)
        for r in (0, n - 1):
            assert np.array_equal(dev.to_host(ds[r], count, npdt).view(np.uint8), want[r].view(np.uint8))
        # what the reference's host loops do not carry is refused, as there
        assert hs.all_reduce(ds, dr, count, dtype, N.OP_PROD)[0] == N.INVALID_ARGUMENT
        assert hs.all_reduce(ds, dr, count, N.DT_BF16, N.OP_SUM)[0] == N.INVALID_ARGUMENT


@pytest.mark.parametrize("dname", ["fp32", "int32", "uint8", "fp64"])
@pytest.mark.parametrize("n,count", [(8, 100003), (3, 10), (4, 2), (5, 77777), (1, 1000)])
def test_host_staged_reduce_and_reduce_scatter_match_host_order_and_oracle(dev, stream, dname, n, count):
    """hostRunnerReduce and hostRunnerReduceScatter end to end (host_runner.cc:12-67,
    291-346 over bootstrap.cc:944-996, 1039-1066): the root's result is the host
    ring's all-reduce result and no other rank's buffer is written; chunk r of a
    reduce-scatter ends on rank r.  Bit for bit the oracle's and what the device
    computes under FX_ORDER_HOST."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    npdt = N.NP_DTYPE[dtype]
    sends = seeded_inputs(dtype, n, count, seed=7 * n + count)
    if dname in ("fp32", "fp64"):
        rng = np.random.default_rng(count + 1)
        sends = [(a * 10.0 ** rng.integers(-3, 9, count)).astype(npdt) for a in sends]
        for i in range(min(count, 3 * n)):
            sends[i % n][i] = (np.nan, 0.0, -0.0)[i % 3]
    with DevBufs(dev) as b, S.HostStaged(n, dev.t.deviceMemcpy) as hs, S.SimGroup(n, order=S.ORDER_HOST) as g:
        ds = [b.put(a) for a in sends]
        dr = [b.alloc(count * es + 16) for _ in range(n)]
        ddev = b.alloc(count * es)
        for op, root in ((N.OP_SUM, n - 1), (N.OP_MAX, 0), (N.OP_MIN, n // 2)):
            want = O.bootstrap_allreduce(sends, dtype, op)[0] if n > 1 else sends[0]
            for q in dr:
                dev.memset(q, 0x5A, count * es + 16)
            rc, _ = hs.reduce(ds, [dr[r] if r == root else None for r in range(n)], count, dtype, op, root)
            N.check(rc, "fxHostStagedReduce")
            N.check(g.reduce(ds, [ddev if r == root else None for r in range(n)], count, dtype, op, root, stream))
            dev.stream_sync(stream)
            got = dev.to_host(dr[root], count, npdt)
            assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(want).view(np.uint8)), f"op {op} vs the oracle"
            assert np.array_equal(got.view(np.uint8), dev.to_host(ddev, count, npdt).view(np.uint8)), f"op {op} vs FX_ORDER_HOST"
            assert (dev.to_host(dr[root] + count * es, 16, np.uint8) == 0x5A).all()
            for r in range(n):
                if r != root:
                    assert (dev.to_host(dr[r], count * es, np.uint8) == 0x5A).all(), "a non-root buffer was written"
        assert hs.reduce(ds, dr, count, dtype, N.OP_SUM, n)[0] == N.INVALID_ARGUMENT
        # reduce-scatter: rank r sends n * rc elements and receives chunk r
        rc_el = max(count // n, 1)
        part = [a[:n * rc_el] if a.size >= n * rc_el else np.resize(a, n * rc_el) for a in sends]
        dp = [b.put(a) for a in part]
        off = (C.c_size_t * n)(*[r * rc_el * es for r in range(n)])
        ln = (C.c_size_t * n)(*[rc_el * es] * n)
        outs = [np.empty(rc_el, npdt) for _ in range(n)]
        vp = lambda arrs: (C.c_void_p * n)(*[a.ctypes.data for a in arrs])
        dd = [b.alloc(rc_el * es) for _ in range(n)]
        for op in (N.OP_SUM, N.OP_MIN):
            if n > 1:
                assert O.lib.oracle_bootstrap_reduce_scatter(vp(outs), vp(part), n, off, ln, dtype, op) == 0
            else:
                outs = [part[0][:rc_el]]
            for q in dr:
                dev.memset(q, 0x5A, count * es + 16)
            rc, _ = hs.reduce_scatter(dp, dr, rc_el, dtype, op)
            N.check(rc, "fxHostStagedReduceScatter")
            N.check(g.reduce_scatter(dp, dd, rc_el, dtype, op, stream))
            dev.stream_sync(stream)
            for r in range(n):
                got = dev.to_host(dr[r], rc_el, npdt)
                assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(outs[r]).view(np.uint8)), f"rank {r} op {op} vs the oracle"
                assert np.array_equal(got.view(np.uint8), dev.to_host(dd[r], rc_el, npdt).view(np.uint8)), f"rank {r} vs FX_ORDER_HOST"
                assert (dev.to_host(dr[r] + rc_el * es, 16, np.uint8) == 0x5A).all(), "wrote past the received chunk"


@pytest.mark.parametrize("n,count,phase", [(9, 1001, 0), (12, 70001, 4), (16, 3, 0), (17, 262147, 8), (33, 4099, 0)])
def test_byte_moving_collectives_over_many_ranks(dev, stream, n, count, phase):
    """Broadcast, gather, scatter and alltoall past eight ranks: every receive
    buffer holds exactly the bytes the definition names, the bytes on either
    side of it stay as they were, and the root may run in place
    (flagcx/adaptor/ccl/rccl_adaptor.cc:126-184,222-246 builds them from
    grouped send/recv pairs)."""
    rng = np.random.default_rng(n * 1000 + count)
    root = (2 * n) // 3
    guard = 64
    fill = np.full(guard, 0xA5, np.uint8)

    def framed(b, nelem, init=None):
        """A device buffer of nelem int32 at `phase` bytes past a guard, with guards on both sides."""
        body = init if init is not None else np.full(nelem, -1, np.int32)
        host = np.concatenate([fill, np.zeros(phase, np.uint8), body.view(np.uint8), fill])
        return b.put(host) + guard + phase

    def check(b, p, want, what):
        got = dev.to_host(p - guard - phase, 2 * guard + phase + want.nbytes, np.uint8)
        assert (got[:guard] == 0xA5).all() and (got[-guard:] == 0xA5).all(), f"{what}: guard bytes written"
        assert np.array_equal(got[guard + phase:-guard].view(np.int32), want), what

    with DevBufs(dev) as b, S.SimGroup(n) as g:
        def each(fn, name):
            for r in range(n):
                N.check(fn(r), name)
            dev.stream_sync(stream)

        # broadcast: out of place everywhere, then in place on the root
        src = [rng.integers(-2**31, 2**31 - 1, count, dtype=np.int32) for _ in range(n)]
        ds = [framed(b, count, src[r]) for r in range(n)]
        dr = [framed(b, count) for _ in range(n)]
        each(lambda r: N.lib.flagcxBroadcast(ds[r], dr[r], count, N.DT_INT32, root, g.comms[r], stream), "flagcxBroadcast")
        for r in range(n):
            check(b, dr[r], src[root], f"broadcast to rank {r}")
            check(b, ds[r], src[r], f"broadcast left rank {r}'s send buffer alone")
        dr2 = [ds[r] if r == root else framed(b, count) for r in range(n)]
        each(lambda r: N.lib.flagcxBroadcast(ds[r], dr2[r], count, N.DT_INT32, root, g.comms[r], stream), "flagcxBroadcast")
        for r in range(n):
            check(b, dr2[r], src[root], f"in-place broadcast to rank {r}")

        # gather to the root, root's own block already in place
        gat = framed(b, n * count)
        gs = [gat + root * count * 4 if r == root else ds[r] for r in range(n)]
        dev.upload(gat + root * count * 4, src[root])
        each(lambda r: N.lib.flagcxGather(gs[r], gat if r == root else None, count, N.DT_INT32, root, g.comms[r], stream),
             "flagcxGather")
        check(b, gat, np.concatenate(src), "gather")

        # scatter the gathered buffer back out
        sc = [framed(b, count) for _ in range(n)]
        each(lambda r: N.lib.flagcxScatter(gat if r == root else None, sc[r], count, N.DT_INT32, root, g.comms[r], stream),
             "flagcxScatter")
        for r in range(n):
            check(b, sc[r], src[r], f"scatter to rank {r}")

        # alltoall: block i of rank r becomes block r of rank i
        blk = max(count // n, 1)
        a2a = [rng.integers(-2**31, 2**31 - 1, n * blk, dtype=np.int32) for _ in range(n)]
        da = [framed(b, n * blk, a2a[r]) for r in range(n)]
        db = [framed(b, n * blk) for _ in range(n)]
        each(lambda r: N.lib.flagcxAlltoAll(da[r], db[r], blk, N.DT_INT32, g.comms[r], stream), "flagcxAlltoAll")
        for i in range(n):
            want = np.concatenate([a2a[r][i * blk:(i + 1) * blk] for r in range(n)])
            check(b, db[i], want, f"alltoall at rank {i}")


def test_progress_tells_a_rank_when_its_collective_has_been_launched(dev, stream):
    """A collective is launched by the last rank that posts it; until then the
    earlier ranks' calls have only been accepted."""
    n, count = 3, 1000
    with DevBufs(dev) as b, S.SimGroup(n) as g:
        bufs = [b.put(np.full(count, r + 1, np.float32)) for r in range(n)]
        assert g.progress(0) == (0, 0)
        for turn in range(2):
            for r in range(n):
                N.check(N.lib.flagcxAllReduce(bufs[r], bufs[r], count, N.DT_FP32, N.OP_SUM, g.comms[r], stream), "flagcxAllReduce")
                joined, launched = g.progress(r)
                assert joined == turn and launched == turn + (r == n - 1)
            assert [g.progress(r) for r in range(n)] == [(turn, turn + 1)] * n
        dev.stream_sync(stream)
        assert (dev.to_host(bufs[0], count, np.float32) == 6 * 3).all()


def test_rendezvous_mode_with_busy_streams_and_no_host_waits(dev):
    """One host thread and one stream per rank, nothing but stream order between
    the steps: every round a rank fills its send buffer on its own stream behind
    a long copy (so the stream is busy when the rank posts), all-reduces, and
    copies the result into that round's slot of a history buffer -- the only
    host wait is at the very end.  A collective that ran before a rank's fill, or
    a result copy that ran before the collective, shows up as a wrong slot."""
    import threading
    n, count, rounds = 6, 1 << 20, 10          # 4 MiB of int32 per rank
    big = 96 << 20
    errors = []
    with DevBufs(dev) as b, S.SimGroup(n, sync=S.SYNC_RENDEZVOUS) as g:
        send = [b.alloc(count * 4) for _ in range(n)]
        recv = [b.alloc(count * 4) for _ in range(n)]
        hist = [b.alloc(rounds * count * 4) for _ in range(n)]
        ballast = [(b.alloc(big), b.alloc(big)) for _ in range(n)]

        def rank_main(r):
            try:
                dev.set_device()
                s = dev.stream_create()
                for it in range(rounds):
                    if (it + r) % 3:                                   # two rounds in three: keep the stream busy
                        dev.copy(ballast[r][1], ballast[r][0], big, s)
                    dev.memset(send[r], (r + 1) * (it + 1) % 41, count * 4, s)     # every byte, so every int32 = 0x01010101 * v
                    N.check(N.lib.flagcxAllReduce(send[r], recv[r], count, N.DT_INT32, N.OP_SUM, g.comms[r], s))
                    dev.copy(hist[r] + it * count * 4, recv[r], count * 4, s)
                dev.stream_sync(s)
                got = dev.to_host(hist[r], rounds * count, np.uint32).reshape(rounds, count)
                for it in range(rounds):
                    want = 0x01010101 * sum((q + 1) * (it + 1) % 41 for q in range(n))
                    if not (got[it] == want).all():
                        errors.append((r, it, hex(int(got[it][0])), hex(want)))
                dev.stream_destroy(s)
            except Exception as e:                      # noqa: BLE001 - reported below
                errors.append((r, repr(e)))

        threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
        assert not any(t.is_alive() for t in threads)
        assert not errors, errors[:6]


@pytest.mark.parametrize("dname", ["bf16", "fp16"])
def test_element_arithmetic_mode_reproduces_the_reference_device_kernel(dev, stream, dname):
    """FX_SIM_ARITH = element: the all-reduce, reduce, reduce-scatter and the
    custom all-reduce hook fold fp16 / bf16 the way lsa_reduce does
    (custom_allreduce.cu:326-361) -- rounded after every addition, max / min
    handing on the later operand -- bit for bit against the oracle's
    restatement; the default mode keeps this build's own contract."""
    dtype = DTYPES[dname]
    n, count = 8, 8 * 12501
    nanbits = 0x7FC0 if dname == "bf16" else 0x7E00
    rng = np.random.default_rng(3)
    sends = seeded_inputs(dtype, n, count, seed=21, dist=(0.0, 300.0))
    for a in sends:
        where = rng.random(count) < 0.01
        a[where] = rng.choice(np.array([0x0000, 0x8000, nanbits], np.uint16), int(where.sum()))
    for op in (N.OP_SUM, N.OP_MAX, N.OP_MIN):
        want = O.reduce_copy_elem(sends, dtype, op)
        plain = O.reduce_copy(sends, dtype, op)
        assert (want != plain).sum() > 100
        nan = (lambda a: is_nan16(a, dtype)) if op == N.OP_SUM else (lambda a: np.zeros(a.shape, bool))

        def same(got, ref, what):
            assert np.array_equal(nan(got), nan(ref)) and np.array_equal(got[~nan(got)], ref[~nan(ref)]), what

        for arith, ref in ((S.ARITH_ELEMENT, want), (S.ARITH_DEFAULT, plain)):
            with DevBufs(dev) as b, S.SimGroup(n, arith=arith) as g:
                ds = [b.put(a) for a in sends]
                dr = [b.alloc(count * 2) for _ in range(n)]
                N.check(g.all_reduce(ds, dr, count, dtype, op, stream), "flagcxAllReduce")
                dev.stream_sync(stream)
                for r in range(n):
                    same(dev.to_host(dr[r], count, np.uint16), ref, f"all-reduce {dname} op={op} arith={arith} rank {r}")
                if arith == S.ARITH_DEFAULT:
                    continue
                rc = count // n
                N.check(g.reduce_scatter(ds, dr, rc, dtype, op, stream), "flagcxReduceScatter")
                N.check(g.reduce(ds, [dr[r] + rc * 2 if r == 5 else None for r in range(n)], count - rc, dtype, op, 5, stream),
                        "flagcxReduce")
                dev.stream_sync(stream)
                for r in range(n):
                    same(dev.to_host(dr[r], rc, np.uint16), want[r * rc:(r + 1) * rc], f"reduce-scatter rank {r}")
                same(dev.to_host(dr[5] + rc * 2, count - rc, np.uint16), want[:count - rc], "reduce to rank 5")
                # the hook, on registered windows
                win = [b.alloc(count * 2) for _ in range(n)]
                N.check(g.register_windows(win, count * 2), "fxSimRegisterWindows")
                N.check(g.custom_all_reduce(ds, dr, count, dtype, op, stream), "flagcxCustomAllReduceImpl")
                dev.stream_sync(stream)
                for r in (0, n - 1):
                    same(dev.to_host(dr[r], count, np.uint16), want, f"custom all-reduce rank {r}")
                # the ring order is not that kernel's schedule: the mode leaves it alone
                g.configure(order=S.ORDER_RING)
                N.check(g.all_reduce(ds, dr, count, dtype, op, stream), "flagcxAllReduce")
                dev.stream_sync(stream)
                ring = np.concatenate([O.reduce_copy([a[lo:hi] for a in sends], dtype, op, first=c)
                                       for c, (lo, hi) in enumerate((c * rc, (c + 1) * rc) for c in range(n))])
                assert_parity(dev.to_host(dr[0], count, np.uint16), ring, dtype, op, "ring order keeps the default arithmetic")
