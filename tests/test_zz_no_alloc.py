"""The entry point that allocates nothing, fx_reduce_slices_static, against the
entry point it is a variant of (fx_plan_create + fx_plan_launch) and against
the CPU oracle: two calls in a row on the same GPU, the second with a smaller
input, so that what the first call left in the static table must not leak into
the second."""
import ctypes as C

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from oracle import fx_oracle as O
from tests.util import DevBufs, assert_parity, seeded_inputs

pytestmark = pytest.mark.gpu

FILL = 0x5A


def _pieces(rng, total, nslices):
    """Non-overlapping (offset, count) pieces of [0, total) with gaps, odd sizes and an empty one."""
    cuts = np.sort(rng.choice(np.arange(1, total), size=2 * nslices - 1, replace=False))
    bounds = np.concatenate([[0], cuts, [total]])
    sl = [(int(bounds[2 * i]), int(bounds[2 * i + 1] - bounds[2 * i])) for i in range(nslices)]
    sl.insert(len(sl) // 2, (sl[0][0], 0))
    return sl


def _both_ways(dev, b, dins, ins, total, sl, k, dtype, op, what):
    """Run the slices through a plan and through the static table into two outputs; both must equal the oracle."""
    es = N.DTYPE_SIZE[dtype]
    outs = [b.alloc(total * es + 64) for _ in range(2)]
    for o in outs:
        dev.memset(o, FILL, total * es + 64)
    descs = [[([p + off * es for p in dins], o + off * es, c) for off, c in sl] for o in outs]
    plan = K.Plan(descs[0], k, dtype, op)
    N.check(plan.launch(), "fx_plan_launch")
    N.check(K.reduce_slices_static(descs[1], k, dtype, op), "fx_reduce_slices_static")
    dev.sync()
    plan.destroy()
    got = [dev.to_host(o, total + 64 // es, N.NP_DTYPE[dtype]) for o in outs]
    want = np.frombuffer(bytes([FILL]) * (total * es + 64), dtype=N.NP_DTYPE[dtype]).copy()
    for off, c in sl:
        if c:
            want[off:off + c] = O.reduce_copy([a[off:off + c] for a in ins], dtype, op)
    assert_parity(got[0], want, dtype, op, f"{what}: plan vs oracle")
    assert_parity(got[1], want, dtype, op, f"{what}: static table vs oracle")
    assert np.array_equal(got[0].view(np.uint8), got[1].view(np.uint8)), f"{what}: static table differs from plan"


@pytest.mark.parametrize("dname,dtype,k,op", [("bf16", N.DT_BF16, 8, N.OP_SUM), ("fp32", N.DT_FP32, 2, N.OP_SUM),
                                              ("int32", N.DT_INT32, 5, N.OP_MAX)])
def test_static_table_equals_plan_twice_second_smaller(dev, dname, dtype, k, op):
    rng = np.random.default_rng(k)
    total = 900_000
    ins = seeded_inputs(dtype, k, total, seed=31)
    with DevBufs(dev) as b:
        dins = [b.put(a) for a in ins]
        # 150 descriptors: five argument blocks of the table writer, ragged, one empty
        _both_ways(dev, b, dins, ins, total, _pieces(rng, total, 150), k, dtype, op, f"{dname} first call")
        # smaller: 7 descriptors over the first 50,000 elements only
        _both_ways(dev, b, dins, ins, 50_000, _pieces(rng, 50_000, 7), k, dtype, op, f"{dname} second call")
        # one large merged segment (pieces that continue each other): the striped hand-out through the table
        chunk = 100_000
        sl = [(i * chunk, chunk) for i in range(total // chunk)]
        _both_ways(dev, b, dins, ins, total, sl, k, dtype, op, f"{dname} third call")


def test_static_table_copy_and_limits(dev):
    total = 300_001
    src = np.random.default_rng(5).integers(0, 256, total, dtype=np.uint8)
    with DevBufs(dev) as b:
        dsrc = b.put(src)
        douts = [b.alloc(total + 64) for _ in range(2)]
        for o in douts:
            dev.memset(o, FILL, total + 64)
        sl = [(0, 1000), (1000, 7), (5003, 100_000), (200_000, 100_001)]
        plan = K.Plan([([dsrc + o], douts[0] + o, c) for o, c in sl], 1, 0, -1)
        N.check(plan.launch(), "fx_plan_launch copy")
        N.check(K.reduce_slices_static([([dsrc + o], douts[1] + o, c) for o, c in sl], 1, 0, -1), "static copy")
        dev.sync()
        plan.destroy()
        got = [dev.to_host(o, total + 64, np.uint8) for o in douts]
        want = np.full(total + 64, FILL, np.uint8)
        for o, c in sl:
            want[o:o + c] = src[o:o + c]
        assert np.array_equal(got[0], want) and np.array_equal(got[1], want)
        # more descriptors than the table holds: rejected, nothing written
        dev.memset(douts[1], FILL, total + 64)
        many = [([dsrc + 2 * i], douts[1] + 2 * i, 1) for i in range(N.STATIC_MAX_SLICES + 1)]
        assert K.reduce_slices_static(many, 1, 0, -1) == N.INVALID_ARGUMENT
        # exactly the limit fits (every second byte, so nothing merges)
        N.check(K.reduce_slices_static(many[:N.STATIC_MAX_SLICES], 1, 0, -1), "static copy at the limit")
        dev.sync()
        got = dev.to_host(douts[1], total + 64, np.uint8)
        want = np.full(total + 64, FILL, np.uint8)
        want[0:2 * N.STATIC_MAX_SLICES:2] = src[0:2 * N.STATIC_MAX_SLICES:2]
        assert np.array_equal(got, want)
    # argument screening as fx_plan_create
    assert K.reduce_slices_static([], 2, N.DT_FP32, N.OP_SUM) == N.SUCCESS
    assert K.reduce_slices_static([([0, 0], 0, 5)], 2, N.DT_FP32, N.OP_SUM) == N.INVALID_ARGUMENT
    assert K.reduce_slices_static([([16, 16], 16, 5)], 9, N.DT_FP32, N.OP_SUM) == N.INVALID_ARGUMENT
    assert K.reduce_slices_static([([16, 16], 16, 5)], 2, 99, N.OP_SUM) == N.INVALID_ARGUMENT


def test_static_table_in_a_captured_graph_two_dependent_calls(dev):
    """What the entry point is for: one eager call first (it looks the table's
    address up), then TWO calls captured on one stream -- different descriptors,
    the second reading what the first wrote, so the second's table overwrites the
    first's while both are in the graph -- replayed on new data; every replay
    against the oracle."""
    hip = C.CDLL("libamdhip64.so.7")          # the runtime the library itself is linked against (same mapping)
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    dtype, op, k, total = N.DT_FP32, N.OP_SUM, 3, 200_003
    rng = np.random.default_rng(11)
    first_sl, second_sl = _pieces(rng, total, 40), _pieces(rng, total, 9)      # 40 descriptors: two table-writer launches
    stream = dev.stream_create()
    raw = dev.raw_stream(stream)
    with DevBufs(dev) as b:
        ins = seeded_inputs(dtype, k, total, seed=3)
        dins = [b.put(a) for a in ins]
        dmid, dout = b.alloc(total * 4), b.alloc(total * 4)
        # the eager call: any call on this GPU outside a capture
        N.check(K.reduce_slices_static([(dins, dmid, 16)], k, dtype, op, raw))
        dev.stream_sync(stream)
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(raw, 0) == 0
        try:
            # mid = in0 + in1 + in2 on the first pieces; out = mid + in0 (two inputs) on the second pieces
            N.check(K.reduce_slices_static([([p + o * 4 for p in dins], dmid + o * 4, c) for o, c in first_sl], k, dtype, op, raw))
            N.check(K.reduce_slices_static([([dmid + o * 4, dins[0] + o * 4], dout + o * 4, c) for o, c in second_sl], 2, dtype,
                                           op, raw))
        finally:
            assert hip.hipStreamEndCapture(raw, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for rep in range(3):
            if rep:
                ins = seeded_inputs(dtype, k, total, seed=3 + rep)
                for d, a in zip(dins, ins):
                    dev.upload(d, a)
            dev.memset(dmid, FILL, total * 4)
            dev.memset(dout, FILL, total * 4)
            # eager work of the program's own between the replays, through the same table
            N.check(K.reduce_slices_static([(dins, dout, 1000)], k, dtype, op, raw))
            dev.stream_sync(stream)
            dev.memset(dout, FILL, total * 4)
            dev.sync()
            assert hip.hipGraphLaunch(gexec, raw) == 0
            dev.stream_sync(stream)
            mid = np.frombuffer(bytes([FILL]) * (total * 4), dtype=np.float32).copy()
            for o, c in first_sl:
                if c:
                    mid[o:o + c] = O.reduce_copy([a[o:o + c] for a in ins], dtype, op)
            want = np.frombuffer(bytes([FILL]) * (total * 4), dtype=np.float32).copy()
            for o, c in second_sl:
                if c:
                    want[o:o + c] = O.reduce2(mid[o:o + c], ins[0][o:o + c], dtype, op)
            assert_parity(dev.to_host(dmid, total, np.float32), mid, dtype, op, f"replay {rep}: first captured call")
            assert_parity(dev.to_host(dout, total, np.float32), want, dtype, op, f"replay {rep}: second captured call")
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
    dev.stream_destroy(stream)
