"""GPU parity of the k-way reduce-copy (through the C ABI) against the CPU
oracle on identical seeded inputs."""
import itertools

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from oracle import fx_oracle as O
from tests.util import DTYPES, OPS, DevBufs, assert_parity, seeded_inputs

pytestmark = pytest.mark.gpu


def run_reduce(dev, ins, dtype, op, first=0, inplace=False, offs=None):
    """Upload ins (optionally at per-buffer byte offsets), reduce on the GPU,
    return the host result."""
    n = ins[0].size
    es = N.DTYPE_SIZE[dtype]
    offs = offs or [0] * (len(ins) + 1)
    with DevBufs(dev) as b:
        dins = [b.put(a, pad_before=o) for a, o in zip(ins, offs[1:])]
        dout = dins[0] if inplace else b.alloc(offs[0] + n * es + 256) + offs[0]
        if not inplace:
            dev.memset(dout - offs[0], 0xA5, offs[0] + n * es + 256)
        N.check(K.reduce_copy(dout, dins, n, dtype, op, first), "fx_reduce_copy")
        dev.sync()
        got = dev.to_host(dout, n, N.NP_DTYPE[dtype])
        if not inplace:  # nothing written past the end
            tail = dev.to_host(dout + n * es, 64, np.uint8)
            assert (tail == 0xA5).all(), "wrote past the end of the output"
    return got


def test_reference_known_answers(dev):
    # test/unittest/service/test_reduction_ops.cpp:11-75
    f = np.float32
    cases = [
        (N.DT_FP32, N.OP_SUM, [1, 2, 3], [4, 5, 6], [5, 7, 9], f),
        (N.DT_INT32, N.OP_SUM, [10, 20, 30], [1, 2, 3], [11, 22, 33], np.int32),
        (N.DT_FP32, N.OP_MIN, [3, 1, 4], [1, 5, 2], [1, 1, 2], f),
        (N.DT_FP32, N.OP_MAX, [3, 1, 4], [1, 5, 2], [3, 5, 4], f),
        (N.DT_FP32, N.OP_SUM, [42], [8], [50], f),
    ]
    for dtype, op, a, b, want, t in cases:
        got = run_reduce(dev, [np.array(a, t), np.array(b, t)], dtype, op)
        assert got.tolist() == want


@pytest.mark.parametrize("dname", list(DTYPES))
@pytest.mark.parametrize("oname", list(OPS))
def test_seeded_parity_k_and_sizes(dev, dname, oname):
    dtype, op = DTYPES[dname], OPS[oname]
    sizes = [1, 3, 8, 63, 1000, 4097, 65536 + 3, (1 << 20) + 5]
    for k, n in itertools.product([1, 2, 3, 4, 5, 6, 7, 8, 9, 17], sizes):
        if k > 8 and n > 70000:
            continue
        ins = seeded_inputs(dtype, k, n, seed=100 + k)
        want = O.reduce_copy(ins, dtype, op)
        got = run_reduce(dev, ins, dtype, op)
        assert_parity(got, want, dtype, op, f"{dname} {oname} k={k} n={n}")


@pytest.mark.parametrize("dname", ["bf16", "fp32", "int8", "uint64"])
def test_largest_input_counts(dev, dname):
    """k = 33 and k = 64 (FX_MAX_INPUTS), rotated, aligned and not, across the
    striped-zone threshold for the wider types."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    for k, n, first, shift in [(33, 70001, 0, 0), (64, 1, 63, 0), (64, 40007, 17, 0), (64, 40007, 0, es),
                               (64, (4 << 20) // es + 5, 5, 0)]:
        ins = seeded_inputs(dtype, k, n, seed=200 + k)
        for op in (N.OP_SUM, N.OP_MAX, N.OP_AVG):
            want = O.reduce_copy(ins, dtype, op, first=first)
            offs = [0] + [shift * (p % 3) for p in range(k)]
            got = run_reduce(dev, ins, dtype, op, first=first, offs=offs)
            assert_parity(got, want, dtype, op, f"{dname} op={op} k={k} n={n} first={first} shift={shift}")


@pytest.mark.parametrize("dname", list(DTYPES))
def test_inplace_matches_out_of_place(dev, dname):
    dtype = DTYPES[dname]
    for op, k, n in itertools.product(OPS.values(), [2, 4, 8], [5, 70001, (1 << 20) + 9]):
        ins = seeded_inputs(dtype, k, n, seed=7)
        want = O.reduce_copy(ins, dtype, op)
        got = run_reduce(dev, ins, dtype, op, inplace=True)
        assert_parity(got, want, dtype, op, f"in-place {dname} op={op} k={k} n={n}")


@pytest.mark.parametrize("dname", list(DTYPES))
def test_rotated_order(dev, dname):
    dtype = DTYPES[dname]
    k, n = 8, 50001
    ins = seeded_inputs(dtype, k, n, seed=11)
    for op in OPS.values():
        for first in (0, 1, 5, 7):
            want = O.reduce_copy(ins, dtype, op, first=first)
            got = run_reduce(dev, ins, dtype, op, first=first)
            assert_parity(got, want, dtype, op, f"{dname} op={op} first={first}")


@pytest.mark.parametrize("dname", list(DTYPES))
def test_unaligned_buffers(dev, dname):
    """Output / inputs at element offsets that are not 16-byte aligned, both
    all-equal (a peeled head, then aligned vectors) and mixed (unaligned vector loads)."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    k = 3
    for n in (1, 2, 9, 255, 5000, 300007):
        ins = seeded_inputs(dtype, k, n, seed=n)
        for offs_el in ([1, 1, 1, 1], [3, 3, 3, 3], [0, 1, 2, 3], [2, 0, 0, 0], [0, 0, 1, 0]):
            offs = [o * es for o in offs_el]
            for op in (N.OP_SUM, N.OP_MAX):
                want = O.reduce_copy(ins, dtype, op)
                got = run_reduce(dev, ins, dtype, op, offs=offs)
                assert_parity(got, want, dtype, op, f"{dname} n={n} offs={offs_el} op={op}")


@pytest.mark.parametrize("dname", ["fp32", "bf16"])
def test_striped_zone_boundaries(dev, dname):
    """Segments a few MiB long handed out as striped regions plus a head and a
    tail: output at odd byte offsets inside its allocation, lengths just around
    whole numbers of 1 MiB regions, in place and out of place, k = 1, 2, 8."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    mib = (1 << 20) // es
    for n, off_el in ((3 * mib, 0), (3 * mib + 1, 0), (2 * mib - 1, 5), (4 * mib + 4097, 131), (mib + 7, mib // 2 + 3),
                      (5 * mib, 4)):
        for k in (1, 2, 8):
            ins = seeded_inputs(dtype, k, n, seed=n % 1000 + k)
            want = O.reduce_copy(ins, dtype, N.OP_SUM)
            offs = [off_el * es] * (k + 1)
            got = run_reduce(dev, ins, dtype, N.OP_SUM, offs=offs)
            assert_parity(got, want, dtype, N.OP_SUM, f"zone {dname} n={n} off={off_el} k={k}")
            got = run_reduce(dev, ins, dtype, N.OP_SUM, offs=offs, inplace=True)
            assert_parity(got, want, dtype, N.OP_SUM, f"zone in-place {dname} n={n} off={off_el} k={k}")
    # inputs NOT co-aligned with the output: no zone, unaligned vector loads over a long segment
    n = 3 * mib + 9
    ins = seeded_inputs(dtype, 3, n, seed=4)
    got = run_reduce(dev, ins, dtype, N.OP_MAX, offs=[0, es, 0, 3 * es])
    assert_parity(got, O.reduce_copy(ins, dtype, N.OP_MAX), dtype, N.OP_MAX, "long gather")


def _special_f32():
    v = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.17549435e-38, 3.4028235e38,
                  -3.4028235e38, 1e8, 1.0, -1e8, 16777216.0, 1.0, 0.5, 1.5, 2.5], np.float32)
    return v


def test_special_values_fp32(dev):
    v = _special_f32()
    grid = np.array(list(itertools.product(v, v, v)), np.float32)  # all triples
    ins = [np.ascontiguousarray(grid[:, j]) for j in range(3)]
    for op in OPS.values():
        want = O.reduce_copy(ins, N.DT_FP32, op)
        got = run_reduce(dev, ins, N.DT_FP32, op)
        if op in (N.OP_SUM, N.OP_PROD, N.OP_AVG):  # NaN payloads of arithmetic are not part of the contract
            gn, wn = np.isnan(got), np.isnan(want)
            assert np.array_equal(gn, wn)
            assert np.array_equal(got[~gn].view(np.uint32), want[~wn].view(np.uint32))
        else:
            assert_parity(got, want, N.DT_FP32, op, f"special fp32 op={op}")


def test_special_values_fp64(dev):
    v = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 5e-324, -5e-324, 2.2250738585072014e-308,
                  1.7976931348623157e308, -1.7976931348623157e308, 1e16, 1.0, -1e16, 9007199254740992.0, 0.5, 1.5,
                  2.5, 1e-310], np.float64)
    grid = np.array(list(itertools.product(v, v, v)), np.float64)
    ins = [np.ascontiguousarray(grid[:, j]) for j in range(3)]
    for op in OPS.values():
        with np.errstate(all="ignore"):
            want = O.reduce_copy(ins, N.DT_FP64, op)
        got = run_reduce(dev, ins, N.DT_FP64, op)
        if op in (N.OP_SUM, N.OP_PROD, N.OP_AVG):
            gn, wn = np.isnan(got), np.isnan(want)
            assert np.array_equal(gn, wn)
            assert np.array_equal(got[~gn].view(np.uint64), want[~wn].view(np.uint64)), op
        else:
            assert_parity(got, want, N.DT_FP64, op, f"special fp64 op={op}")


@pytest.mark.parametrize("dname", ["bf16", "fp16"])
def test_all_16bit_patterns(dev, dname):
    """Every 16-bit pattern (incl. NaNs, infinities, subnormals, +-0) against
    shuffled copies of itself."""
    dtype = DTYPES[dname]
    allbits = np.arange(65536, dtype=np.uint16)
    rng = np.random.default_rng(5)
    ins = [allbits] + [rng.permutation(allbits) for _ in range(3)]
    for op in OPS.values():
        want = O.reduce_copy(ins, dtype, op)
        got = run_reduce(dev, ins, dtype, op)
        assert_parity(got, want, dtype, op, f"all {dname} patterns op={op}")
    # pairs around rounding ties: x + tiny
    for op in (N.OP_SUM, N.OP_PROD):
        a = np.repeat(allbits[::7], 8)
        b = np.tile(np.array([0x0001, 0x8001, 0x3c00, 0x3f80, 0x0400, 0x0080, 0x7bff, 0x7f7f], np.uint16),
                    a.size // 8)
        want = O.reduce_copy([a, b], dtype, op)
        got = run_reduce(dev, [a, b], dtype, op)
        assert_parity(got, want, dtype, op, f"{dname} ties op={op}")


def test_int32_wraparound(dev):
    a = np.array([2**31 - 1, -2**31, 123456789, -1, 65536, 46341], np.int32)
    b = np.array([1, -1, 987654321, -2**31, 65536, 46341], np.int32)
    c = np.array([2**31 - 1, -2**31, 2, 2, 3, 2], np.int32)
    for op in OPS.values():
        want = O.reduce_copy([a, b, c], N.DT_INT32, op)
        got = run_reduce(dev, [a, b, c], N.DT_INT32, op)
        assert_parity(got, want, N.DT_INT32, op, f"int32 wrap op={op}")
    s = run_reduce(dev, [a, b, c], N.DT_INT32, N.OP_SUM).astype(np.int64)
    assert np.array_equal(s, ((a.astype(np.int64) + b + c + 2**31) % 2**32) - 2**31)


def test_error_paths(dev):
    p = dev.malloc(64)
    try:
        ok = lambda dtype, op, k=2, first=0, out=p, ins=None, n=4: K.reduce_copy(out, ins or [p] * k, n, dtype, op, first)
        assert ok(N.DT_FP32, N.OP_SUM) == N.SUCCESS
        assert ok(N.DT_FP32, N.OP_AVG) == N.SUCCESS             # every FlagCX type and op is carried
        assert ok(10, N.OP_SUM) == N.INVALID_ARGUMENT           # outside the enums
        assert ok(N.DT_FP32, 5) == N.INVALID_ARGUMENT
        assert ok(N.DT_FP32, N.OP_SUM, first=2) == N.INVALID_ARGUMENT
        assert ok(N.DT_FP32, N.OP_SUM, out=None) == N.INVALID_ARGUMENT
        assert ok(N.DT_FP32, N.OP_SUM, out=p + 2) == N.INVALID_ARGUMENT   # not element aligned
        assert ok(N.DT_FP32, N.OP_SUM, ins=[p, None]) == N.INVALID_ARGUMENT
        assert K.reduce_copy(p, [p] * 65, 4, N.DT_FP32, N.OP_SUM) == N.INVALID_ARGUMENT
        assert K.reduce_copy(None, [None], 0, N.DT_FP32, N.OP_SUM) == N.SUCCESS  # empty input
        dev.sync()
    finally:
        dev.free(p)


def test_concurrent_host_threads(dev):
    """The C ABI is enqueue-only and thread-safe: four host threads launch on
    their own streams at the same time (ctypes drops the GIL around each call)."""
    import threading
    jobs = [(N.DT_BF16, N.OP_SUM, 8, 300007), (N.DT_FP32, N.OP_MAX, 3, 70001), (N.DT_INT64, N.OP_PROD, 2, 65537),
            (N.DT_UINT8, N.OP_SUM, 5, 1 << 20)]
    errors, results = [], {}
    with DevBufs(dev) as b:
        prepared = []
        for dtype, op, k, n in jobs:
            ins = seeded_inputs(dtype, k, n, seed=k)
            prepared.append((dtype, op, n, ins, [b.put(a) for a in ins], b.alloc(n * N.DTYPE_SIZE[dtype])))

        def work(i):
            try:
                dev.set_device()
                dtype, op, n, _, dins, dout = prepared[i]
                s = dev.stream_create()
                for _ in range(50):
                    N.check(K.reduce_copy(dout, dins, n, dtype, op, 0, dev.raw_stream(s)), "fx_reduce_copy")
                dev.stream_sync(s)
                results[i] = dev.to_host(dout, n, N.NP_DTYPE[dtype])
                dev.stream_destroy(s)
            except Exception as e:                      # noqa: BLE001 - reported below
                errors.append((i, repr(e)))

        threads = [threading.Thread(target=work, args=(i,)) for i in range(len(jobs))]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=60)
        assert not errors, errors
        for i, (dtype, op, n, ins, _, _) in enumerate(prepared):
            assert_parity(results[i], O.reduce_copy(ins, dtype, op), dtype, op, f"thread {i}")
