"""The entry point that allocates nothing, fx_reduce_slices_static, against the
entry point it is a variant of (fx_plan_create + fx_plan_launch) and against
the CPU oracle: two calls in a row on the same GPU, the second with a smaller
input, so that what the first call left in the static table must not leak into
the second."""
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
