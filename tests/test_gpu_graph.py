"""The enqueue-only entry points inside a captured HIP graph: what a caller that
replays its step as a graph gets.  The graph is replayed several times with the
program's own eager work and synchronisations between the replays, and every
replay is compared with the oracle on the inputs it ran on."""
import ctypes as C

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from oracle import fx_oracle as O
from tests.util import DevBufs, assert_parity, seeded_inputs

pytestmark = pytest.mark.gpu

hip = C.CDLL("libamdhip64.so.7")          # the runtime the library itself is linked against (same mapping)
hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
hip.hipGraphDestroy.argtypes = [C.c_void_p]


def test_reduce_entry_points_replay_correctly_in_a_graph(dev):
    k, n = 8, 300007
    dtype, op = N.DT_BF16, N.OP_SUM
    stream = dev.stream_create()
    raw = dev.raw_stream(stream)
    with DevBufs(dev) as b:
        ins = seeded_inputs(dtype, k, n, seed=1)
        dins = [b.put(a) for a in ins]
        dsum, dmax, dcopy = b.alloc(n * 2), b.alloc(n * 2), b.alloc(n * 2)
        douts = [b.alloc(n * 2) for _ in range(3)]
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(raw, 0) == 0                                  # hipStreamCaptureModeGlobal
        try:
            N.check(K.reduce_copy(dsum, dins, n, dtype, op, 0, raw))                    # direct kernel
            half = n // 2                                                               # two slices with a gap in the table
            N.check(K.reduce_slices([(dins[:2], dmax, half - 1), ([p + 2 * half for p in dins[:2]], dmax + 2 * half, n - half)],
                                    2, dtype, N.OP_MAX, raw))                            # kernel-argument table
            N.check(K.copy_slices([(dsum, dcopy, n * 2)], raw))                         # depends on the first node
            N.check(K.reduce_bcast_slices([(dins, douts, n)], k, 3, dtype, N.OP_AVG, raw))
        finally:
            assert hip.hipStreamEndCapture(raw, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for rep in range(4):
            if rep:                                   # eager work between replays: new inputs, scrubbed outputs
                ins = seeded_inputs(dtype, k, n, seed=1 + rep)
                for d, a in zip(dins, ins):
                    dev.upload(d, a)
                for d in [dsum, dmax, dcopy] + douts:
                    dev.memset(d, 0xEE, n * 2)
                dev.sync()
            assert hip.hipGraphLaunch(gexec, raw) == 0
            dev.stream_sync(stream)
            want = O.reduce_copy(ins, dtype, op)
            assert_parity(dev.to_host(dsum, n, np.uint16), want, dtype, op, f"replay {rep} sum")
            assert np.array_equal(dev.to_host(dcopy, n, np.uint16), dev.to_host(dsum, n, np.uint16))
            wmax = O.reduce_copy(ins[:2], dtype, N.OP_MAX)
            wmax[half - 1] = 0xEEEE if rep else dev.to_host(dmax + 2 * (half - 1), 1, np.uint16)[0]   # the gap is not written
            assert_parity(dev.to_host(dmax, n, np.uint16), wmax, dtype, N.OP_MAX, f"replay {rep} max")
            avg = O.reduce_copy(ins, dtype, N.OP_AVG)
            for d in douts:
                assert_parity(dev.to_host(d, n, np.uint16), avg, dtype, N.OP_AVG, f"replay {rep} avg")
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
    dev.stream_destroy(stream)


def test_simulated_rank_allreduce_replays_correctly_in_a_graph(dev):
    """All ranks post on the one captured stream, so the collective is a single
    kernel node (no events, no scratch): an 8-rank all-reduce and a reduce-scatter
    captured once, replayed on new data."""
    from flagcx_amd import sim as S
    n, count = 8, 8 * 40001
    dtype = N.DT_FP32
    stream = dev.stream_create()
    raw = dev.raw_stream(stream)
    with DevBufs(dev) as b, S.SimGroup(n) as g:
        sends = seeded_inputs(dtype, n, count, seed=3)
        ds = [b.put(a) for a in sends]
        dr = [b.alloc(count * 4) for _ in range(n)]
        dp = [b.alloc(count // n * 4) for _ in range(n)]
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(raw, 0) == 0
        try:
            N.check(g.all_reduce(ds, dr, count, dtype, N.OP_SUM, stream))
            N.check(g.reduce_scatter(ds, dp, count // n, dtype, N.OP_MAX, stream))
        finally:
            assert hip.hipStreamEndCapture(raw, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for rep in range(3):
            if rep:
                sends = seeded_inputs(dtype, n, count, seed=3 + rep)
                for d, a in zip(ds, sends):
                    dev.upload(d, a)
                for d in dr:
                    dev.memset(d, 0xEE, count * 4)
                dev.sync()
            assert hip.hipGraphLaunch(gexec, raw) == 0
            dev.stream_sync(stream)
            want = O.reduce_copy(sends, dtype, N.OP_SUM)
            wmax = O.reduce_copy(sends, dtype, N.OP_MAX)
            for r in (0, 3, n - 1):
                assert_parity(dev.to_host(dr[r], count, np.float32), want, dtype, N.OP_SUM, f"replay {rep} rank {r}")
                part = count // n
                assert_parity(dev.to_host(dp[r], part, np.float32), wmax[r * part:(r + 1) * part], dtype, N.OP_MAX,
                              f"replay {rep} reduce-scatter rank {r}")
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
    dev.stream_destroy(stream)


def test_scratch_users_capture_cold_after_a_reservation(dev):
    """Ring reduce-scatter, in-place all-to-all and the tree-order reduce of more
    than eight ranks need scratch.
    With the scratch reserved at set-up (fxSimCommConfig FX_SIM_SCRATCH_BYTES) their
    very first call may be inside a capture -- no eager call beforehand -- and the
    graph replays correctly on new data; without a reservation the same call is
    refused while the stream is capturing, and works eagerly afterwards."""
    from flagcx_amd import sim as S
    n, count = 5, 5 * 30011
    dtype = N.DT_FP32
    stream = dev.stream_create()
    raw = dev.raw_stream(stream)
    with DevBufs(dev) as b:
        sends = seeded_inputs(dtype, n, count, seed=8)
        ds = [b.put(a) for a in sends]
        droot = b.alloc(count * 4)
        dp = [b.alloc(count // n * 4) for _ in range(n)]
        da = [b.put(a) for a in sends]                       # all-to-all runs in place on these
        graph, gexec = C.c_void_p(), C.c_void_p()
        # no reservation: a call that needs scratch is refused under capture (nothing is enqueued), fine eagerly;
        # the tree-order reduce of up to eight ranks keeps its partials in registers and needs none
        with S.SimGroup(n, order=S.ORDER_TREE, algo=S.ALGO_RING) as g:
            assert hip.hipStreamBeginCapture(raw, 0) == 0
            try:
                rc = g.reduce_scatter(ds, dp, count // n, dtype, N.OP_SUM, stream)
                rc_tree = g.reduce(ds, [droot] * n, count, dtype, N.OP_SUM, 2, stream)
            finally:
                assert hip.hipStreamEndCapture(raw, C.byref(graph)) == 0
            assert rc == N.INVALID_USAGE and rc_tree == N.SUCCESS
            hip.hipGraphDestroy(graph)
            N.check(g.reduce(ds, [droot] * n, count, dtype, N.OP_SUM, 2, stream))
            N.check(g.reduce_scatter(ds, dp, count // n, dtype, N.OP_SUM, stream))
            dev.stream_sync(stream)
            assert_parity(dev.to_host(droot, count, np.float32), O.tree_reduce(sends, 2, dtype, N.OP_SUM), dtype,
                          N.OP_SUM, "eager tree reduce")
        # reserved: cold capture
        with S.SimGroup(n, order=S.ORDER_TREE, algo=S.ALGO_RING, scratch_bytes=n * n * count * 4) as g:
            assert hip.hipStreamBeginCapture(raw, 0) == 0
            try:
                N.check(g.reduce(ds, [droot] * n, count, dtype, N.OP_SUM, 2, stream))
                N.check(g.reduce_scatter(ds, dp, count // n, dtype, N.OP_SUM, stream))
                N.check(N.lib.flagcxAlltoAll(da[0], da[0], count // n, dtype, g.comms[0], stream))
                for r in range(1, n):
                    N.check(N.lib.flagcxAlltoAll(da[r], da[r], count // n, dtype, g.comms[r], stream))
            finally:
                assert hip.hipStreamEndCapture(raw, C.byref(graph)) == 0
            assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
            part = count // n
            for rep in range(3):
                if rep:
                    sends = seeded_inputs(dtype, n, count, seed=8 + rep)
                    for d, a in zip(ds, sends):
                        dev.upload(d, a)
                for d, a in zip(da, sends):
                    dev.upload(d, a)
                dev.memset(droot, 0xEE, count * 4)
                dev.sync()
                assert hip.hipGraphLaunch(gexec, raw) == 0
                dev.stream_sync(stream)
                assert_parity(dev.to_host(droot, count, np.float32), O.tree_reduce(sends, 2, dtype, N.OP_SUM), dtype,
                              N.OP_SUM, f"replay {rep} tree reduce")
                for r in (0, n - 1):
                    # the ring leaves chunk r on rank r folded from rank r + 1 round to rank r
                    want = O.reduce_copy([a[r * part:(r + 1) * part] for a in sends], dtype, N.OP_SUM, first=(r + 1) % n)
                    assert_parity(dev.to_host(dp[r], part, np.float32), want, dtype, N.OP_SUM,
                                  f"replay {rep} reduce-scatter rank {r}")
                    a2a = dev.to_host(da[r], count, np.float32)
                    for src in range(n):
                        assert np.array_equal(a2a[src * part:(src + 1) * part].view(np.uint32),
                                              sends[src][r * part:(r + 1) * part].view(np.uint32)), (rep, r, src)
            hip.hipGraphExecDestroy(gexec)
            hip.hipGraphDestroy(graph)
    dev.stream_destroy(stream)
