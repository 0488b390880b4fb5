"""Pins the CPU oracle: reference known-answer vectors, independent IEEE /
integer implementations (numpy), exhaustive conversion tables, brute force on
tiny inputs, and invariants of the partition / pack arithmetic.  No GPU."""
import itertools

import numpy as np
import pytest

from oracle import fx_oracle as O

I32, F16, F32, BF16 = 2, 6, 7, 9
SUM, PROD, MAX, MIN = 0, 1, 2, 3


# ---- reference KATs: test/unittest/service/test_reduction_ops.cpp:11-75 -------------
def test_reference_known_answers():
    f = np.float32
    assert O.reduce2(np.array([1, 2, 3], f), np.array([4, 5, 6], f), F32, SUM).tolist() == [5, 7, 9]
    assert O.reduce2(np.array([10, 20, 30], np.int32), np.array([1, 2, 3], np.int32), I32, SUM).tolist() == [11, 22, 33]
    assert O.reduce2(np.array([3, 1, 4], f), np.array([1, 5, 2], f), F32, MIN).tolist() == [1, 1, 2]
    assert O.reduce2(np.array([3, 1, 4], f), np.array([1, 5, 2], f), F32, MAX).tolist() == [3, 5, 4]
    assert O.reduce2(np.array([42], f), np.array([8], f), F32, SUM).tolist() == [50]


# ---- fp32 / int32 arithmetic against numpy (independent correctly rounded implementation) ----
def _rand_f32(rng, n):
    mant = rng.standard_normal(n).astype(np.float32)
    return mant * np.float32(2.0) ** rng.integers(-30, 30, n).astype(np.float32)


@pytest.mark.parametrize("k", [2, 3, 5, 8])
def test_fp32_left_fold_matches_numpy(k):
    rng = np.random.default_rng(k)
    ins = [_rand_f32(rng, 20000) for _ in range(k)]
    acc_s, acc_p, acc_mx, acc_mn = (ins[0].copy() for _ in range(4))
    old = np.seterr(all="ignore")
    for x in ins[1:]:
        acc_s = acc_s + x                      # float32 + float32, IEEE RNE
        acc_p = acc_p * x
        acc_mx = np.where(acc_mx < x, x, acc_mx)
        acc_mn = np.where(x < acc_mn, x, acc_mn)
    np.seterr(**old)
    if True:
        for op, want in ((SUM, acc_s), (PROD, acc_p), (MAX, acc_mx), (MIN, acc_mn)):
            got = O.reduce_copy(ins, F32, op)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), op


def test_order_is_left_to_right_not_any_other_parenthesisation():
    # (1e8 + 1) - 1e8 + 1 in fp32: left fold gives 1.0 ; right fold gives 0.0 ; pairwise gives 1.0/0.0 mixes
    f = np.float32
    ins = [np.array([v], f) for v in (1e8, 1.0, -1e8, 1.0)]
    got = O.reduce_copy(ins, F32, SUM)[0]
    left = f(f(f(f(1e8) + f(1.0)) + f(-1e8)) + f(1.0))
    right = f(f(1e8) + f(f(1.0) + f(f(-1e8) + f(1.0))))
    pair = f(f(f(1e8) + f(1.0)) + f(f(-1e8) + f(1.0)))
    assert got == left == 1.0
    assert right != left and pair != left
    # rotation: first=1 -> ((1 + -1e8) + 1) + 1e8
    rot = O.reduce_copy(ins, F32, SUM, first=1)[0]
    assert rot == f(f(f(f(1.0) + f(-1e8)) + f(1.0)) + f(1e8))


def test_brute_force_orders_tiny():
    """For every permutation of a non-associative 4-tuple, oracle(first=0) on the
    permuted inputs equals the explicit left fold."""
    f = np.float32
    vals = [f(16777216.0), f(1.0), f(1.0), f(-16777216.0)]
    for perm in itertools.permutations(range(4)):
        ins = [np.array([vals[i]], f) for i in perm]
        acc = ins[0][0]
        for x in ins[1:]:
            acc = f(acc + x[0])
        assert O.reduce_copy(ins, F32, SUM)[0] == acc


def test_int32_wraps_modulo_2_32():
    rng = np.random.default_rng(0)
    ins = [rng.integers(-2**31, 2**31, 5000, dtype=np.int64).astype(np.int32) for _ in range(4)]
    wide_s = sum(a.astype(np.int64) for a in ins)
    want_s = ((wide_s + 2**31) % 2**32 - 2**31).astype(np.int32)
    assert np.array_equal(O.reduce_copy(ins, I32, SUM), want_s)
    prod = np.ones(5000, dtype=object)
    for a in ins:
        prod = prod * a.astype(object)
    want_p = np.array([((int(v) + 2**31) % 2**32) - 2**31 for v in prod], np.int32)
    assert np.array_equal(O.reduce_copy(ins, I32, PROD), want_p)
    assert np.array_equal(O.reduce_copy(ins, I32, MAX), np.maximum.reduce(ins))
    assert np.array_equal(O.reduce_copy(ins, I32, MIN), np.minimum.reduce(ins))
    # cfg3's int32 prod overflows: 4 values up to 2^20
    big = [np.array([1 << 20], np.int32)] * 4
    assert O.reduce_copy(big, I32, PROD)[0] == 0


def test_max_min_tie_and_nan_rules():
    f = np.float32
    pz, nz, nan = f(0.0), f(-0.0), f(np.nan)
    bits = lambda a: a.view(np.uint32)[0]
    # std::max(a,b) = (a<b)?b:a keeps a on ties; NaN comparisons are false -> keep a
    assert bits(O.reduce2(np.array([pz]), np.array([nz]), F32, MAX)) == 0x00000000
    assert bits(O.reduce2(np.array([nz]), np.array([pz]), F32, MAX)) == 0x80000000
    assert bits(O.reduce2(np.array([pz]), np.array([nz]), F32, MIN)) == 0x00000000
    assert O.reduce2(np.array([f(1)]), np.array([nan]), F32, MAX)[0] == 1.0
    assert np.isnan(O.reduce2(np.array([nan]), np.array([f(1)]), F32, MAX)[0])
    assert O.reduce2(np.array([f(1)]), np.array([nan]), F32, MIN)[0] == 1.0


# ---- 16-bit conversions: exhaustive against numpy / arithmetic definitions --------------
def test_f16_widening_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([O.lib.oracle_f16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_bf16_widening_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = (bits.astype(np.uint32) << 16).view(np.float32)
    got = np.array([O.lib.oracle_bf16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)        # a NaN's payload does not survive the trip through a Python float
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def _probe_floats():
    """fp32 values around every fp16 / bf16 rounding boundary plus random ones."""
    rng = np.random.default_rng(1)
    h = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid16 = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)   # exact ties
    b = (np.arange(0, 0x7f80, 7, dtype=np.uint32) << 16).view(np.float32)
    midb = ((b.view(np.uint32) | 0x8000)).view(np.float32)                                   # bf16 ties
    rnd = rng.integers(0, 2**32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    base = np.concatenate([h, mid16, np.nextafter(mid16, np.float32(np.inf)), np.nextafter(mid16, np.float32(0)),
                           b, midb, np.nextafter(midb, np.float32(np.inf)), np.nextafter(midb, np.float32(0)), rnd,
                           np.array([65504, 65519.996, 65520, 65536, 1e30, np.inf, 5.9604645e-08, 2.9802322e-08,
                                     2.9802326e-08, 1e-10, 0], np.float32)])
    return np.concatenate([base, -base])


def test_f32_to_f16_matches_numpy_rne():
    x = _probe_floats()
    with np.errstate(all="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([O.lib.oracle_f32_to_f16(float(v)) for v in x], np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7c00) == 0x7c00).all() and ((got[nan] & 0x3ff) != 0).all()


def test_f32_to_bf16_is_rne_by_definition():
    """Second, arithmetic implementation: pick the nearer of the two bf16
    neighbours in exact (float64) arithmetic, ties to the even pattern."""
    x = _probe_floats()
    x = x[np.isfinite(x)]
    got = np.array([O.lib.oracle_f32_to_bf16(float(v)) for v in x], np.uint16)
    u = x.view(np.uint32)
    lo = (u & 0xffff0000)
    hi = lo + 0x10000                                   # next pattern away from zero (may be inf)
    flo, fhi = lo.view(np.float32).astype(np.float64), hi.astype(np.uint32).view(np.float32).astype(np.float64)
    xd = x.astype(np.float64)
    with np.errstate(all="ignore"):
        dlo, dhi = np.abs(xd - flo), np.abs(fhi - xd)
    # overflow past the largest finite: the "hi" neighbour is infinity whose virtual value is 2^128
    hi_inf = (hi & 0x7fffffff) == 0x7f800000
    dhi = np.where(hi_inf, np.abs(np.float64(2.0) ** 128 - np.abs(xd)), dhi)
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (((lo >> 16) & 1) == 1))
    want = np.where(pick_hi, hi >> 16, lo >> 16).astype(np.uint16)
    assert np.array_equal(got, want)
    assert O.lib.oracle_f32_to_bf16(float("nan")) & 0x7fc0 == 0x7fc0


@pytest.mark.parametrize("dtype", [BF16, F16])
def test_16bit_sum_within_one_ulp_of_fp64_accumulation(dtype):
    rng = np.random.default_rng(3)
    k, n = 8, 50000
    vals = [rng.standard_normal(n).astype(np.float32) for _ in range(k)]
    if dtype == F16:
        ins = [v.astype(np.float16).view(np.uint16) for v in vals]
        wide = [b.view(np.float16).astype(np.float64) for b in ins]
        to16 = lambda d: d.astype(np.float16).view(np.uint16)
    else:
        ins = [((v.view(np.uint32) + 0x7fff + ((v.view(np.uint32) >> 16) & 1)) >> 16).astype(np.uint16) for v in vals]
        wide = [(b.astype(np.uint32) << 16).view(np.float32).astype(np.float64) for b in ins]
        to16 = lambda d: np.array([O.lib.oracle_f32_to_bf16(float(np.float32(x))) for x in d], np.uint16)
    got = O.reduce_copy(ins, dtype, SUM)
    exact = to16(sum(wide))
    order = lambda b: np.where(b & 0x8000, -(b & 0x7fff).astype(np.int32), (b & 0x7fff).astype(np.int32))
    assert np.abs(order(got) - order(exact)).max() <= 1
    # and exactly equal to an fp32 left fold rounded once (the contract)
    acc = (wide[0]).astype(np.float32)
    for w in wide[1:]:
        acc = acc + w.astype(np.float32)
    assert np.array_equal(got, to16(acc) if dtype == F16 else
                          np.array([O.lib.oracle_f32_to_bf16(float(x)) for x in acc], np.uint16))


def test_16bit_max_min_return_input_bits():
    allb = np.arange(65536, dtype=np.uint16)
    rng = np.random.default_rng(9)
    other = rng.permutation(allb)
    for dtype, widen in ((F16, lambda b: b.view(np.float16).astype(np.float32)),
                         (BF16, lambda b: (b.astype(np.uint32) << 16).view(np.float32))):
        a, b = widen(allb), widen(other)
        with np.errstate(invalid="ignore"):
            want_max = np.where(a < b, other, allb)
            want_min = np.where(b < a, other, allb)
        assert np.array_equal(O.reduce_copy([allb, other], dtype, MAX), want_max)
        assert np.array_equal(O.reduce_copy([allb, other], dtype, MIN), want_min)


def test_host_ring_passes_equal_kway_for_exact_types():
    rng = np.random.default_rng(4)
    ins = [_rand_f32(rng, 3000) for _ in range(6)]
    for op in (SUM, MAX, MIN, PROD):
        with np.errstate(all="ignore"):
            a = O.host_ring_passes(ins, F32, op)
            b = O.reduce_copy(ins, F32, op)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_unsupported_arguments_are_rejected():
    a = np.zeros(4, np.float32)
    for dtype, op in ((10, SUM), (-1, SUM), (F32, 5), (F32, -1)):   # outside the enums
        with pytest.raises(ValueError):
            O.reduce2(a, a, dtype, op)


# ---- the other element types of the host dispatch (utils.h:664-695) --------------------------
_HOST_INTS = {0: np.int8, 1: np.uint8, 3: np.uint32, 4: np.int64, 5: np.uint64}


@pytest.mark.parametrize("dtype", sorted(_HOST_INTS))
def test_host_integer_types_match_numpy_of_the_same_width(dtype):
    """numpy's fixed-width integer arrays wrap on overflow like the C loops do;
    extremes and equal values are planted so that wrap and ties are exercised."""
    t = np.dtype(_HOST_INTS[dtype])
    lo, hi = np.iinfo(t).min, np.iinfo(t).max
    rng = np.random.default_rng(dtype)
    for k in (1, 2, 3, 8):
        ins = [rng.integers(lo, hi, 4000, dtype=t, endpoint=True) for _ in range(k)]
        for a in ins:
            a[:4] = [hi, lo, hi, 0]
        ins[-1][4:8] = ins[0][4:8]
        with np.errstate(over="ignore"):
            want = {SUM: ins[0].copy(), PROD: ins[0].copy(), MAX: ins[0].copy(), MIN: ins[0].copy()}
            for x in ins[1:]:
                want[SUM] = (want[SUM] + x).astype(t)
                want[PROD] = (want[PROD] * x).astype(t)
                want[MAX] = np.maximum(want[MAX], x)
                want[MIN] = np.minimum(want[MIN], x)
        for op in (SUM, PROD, MAX, MIN):
            assert np.array_equal(O.reduce_copy(ins, dtype, op), want[op]), (dtype, k, op)
    # closed forms: hi + 1 wraps to lo; 2^(bits-1) * 2 wraps to 0; big-int arithmetic modulo 2^bits
    one, top = np.array([1], t), np.array([hi], t)
    assert O.reduce_copy([top, one], dtype, SUM)[0] == lo
    bits = 8 * t.itemsize
    vals = [int(x) for x in rng.integers(lo, hi, 5, dtype=t, endpoint=True)]
    p = 1
    for v in vals:
        p *= v
    p %= 1 << bits
    if lo < 0 and p >= 1 << (bits - 1):
        p -= 1 << bits
    assert int(O.reduce_copy([np.array([v], t) for v in vals], dtype, PROD)[0]) == p


def test_fp64_left_fold_matches_numpy():
    rng = np.random.default_rng(8)
    for k in (1, 2, 5, 8):
        ins = [rng.uniform(-1, 1, 3000) * 10.0 ** rng.integers(-20, 20, 3000) for _ in range(k)]
        ins[0][:4] = [0.0, -0.0, np.nan, 1.0]
        if k > 1:
            ins[1][:4] = [-0.0, 0.0, 1.0, np.nan]
        acc = {op: ins[0].copy() for op in (SUM, PROD, MAX, MIN)}
        with np.errstate(all="ignore"):
            for x in ins[1:]:
                acc[SUM] = acc[SUM] + x
                acc[PROD] = acc[PROD] * x
                acc[MAX] = np.where(acc[MAX] < x, x, acc[MAX])
                acc[MIN] = np.where(x < acc[MIN], x, acc[MIN])
            for op in (SUM, PROD, MAX, MIN):
                got = O.reduce_copy(ins, 8, op)
                nan = np.isnan(acc[op])
                assert np.array_equal(np.isnan(got), nan)
                assert np.array_equal(got.view(np.uint64)[~nan], acc[op].view(np.uint64)[~nan]), (k, op)
    # order: a triple whose left fold differs from the right fold in double precision
    a, b, c = np.array([1e16]), np.array([1.0]), np.array([-1e16])
    assert O.reduce_copy([a, b, c], 8, SUM)[0] == 0.0 and O.reduce_copy([a, c, b], 8, SUM)[0] == 1.0


# ---- the host ring (service/bootstrap.cc:787-942) --------------------------------------------
def test_bootstrap_chunk_table():
    # literal evaluations of ceil(size / n) rounded up to the element size, offsets clamped to size
    assert O.bootstrap_chunks(40, 3, 4) == ([0, 16, 32], [16, 16, 8])          # 10 floats over 3 ranks: 4, 4, 2
    assert O.bootstrap_chunks(8, 4, 4) == ([0, 4, 8, 8], [4, 4, 0, 0])          # fewer elements than ranks
    assert O.bootstrap_chunks(7, 3, 1) == ([0, 3, 6], [3, 3, 1])
    assert O.bootstrap_chunks(0, 2, 4) == ([0, 0], [0, 0])
    assert O.bootstrap_chunks(64, 8, 8) == ([8 * i for i in range(8)], [8] * 8)
    for size_el, n, ts in itertools.product((1, 5, 17, 1000, 1001), (1, 2, 3, 8), (1, 2, 4, 8)):
        off, ln = O.bootstrap_chunks(size_el * ts, n, ts)
        assert sum(ln) == size_el * ts and all(x % ts == 0 for x in off + ln)
        assert all(off[i] + ln[i] == off[i + 1] for i in range(n - 1) if ln[i + 1]) and off[0] == 0


def test_bootstrap_ring_association_derived_by_hand():
    """Reading the loop at bootstrap.cc:805-871: chunk c starts on rank c+1 and
    every later rank computes local + received, so rank c ends with
    x_c + (x_{c-1} + (.. (x_{c+2} + x_{c+1}))).  The values make every other
    association (rank order, the uniRunner ring's rotation, pairwise) differ."""
    f = np.float32
    for n in (3, 4):
        per = 50
        count = per * n                                      # chunk c = elements [50 c, 50 c + 50)
        rng = np.random.default_rng(n)
        sends = [(rng.uniform(-1, 1, count) * 10.0 ** rng.integers(-3, 9, count)).astype(f) for _ in range(n)]
        want = np.empty(count, f)
        for c in range(n):
            sl = slice(per * c, per * (c + 1))
            acc = sends[(c + 1) % n][sl]
            for j in range(2, n + 1):
                acc = sends[(c + j) % n][sl] + acc           # local + received
            want[sl] = acc
        got = O.bootstrap_allreduce(sends, F32, SUM)
        for r in range(n):
            assert np.array_equal(got[r].view(np.uint32), want.view(np.uint32)), (n, r)
        assert not np.array_equal(O.reduce_copy(sends, F32, SUM).view(np.uint32), want.view(np.uint32))
        ring = O.ring_allreduce(sends, F32, SUM)[0]
        assert not np.array_equal(ring.view(np.uint32), want.view(np.uint32))
    # max / min return the LOCAL operand unless strictly beaten ((a < b) ? b : a, utils.h:707-725), so among
    # zeros of either sign the last rank of the chain -- rank c for chunk c -- decides
    n, count = 3, 6
    pz, nz = f(0.0), f(-0.0)
    sends = [np.array([pz, nz, nz, pz, nz, pz], f), np.array([nz, nz, pz, pz, pz, nz], f), np.array([nz, pz, pz, nz, nz, nz], f)]
    for op in (MAX, MIN):
        got = O.bootstrap_allreduce(sends, F32, op)[0]
        want = np.concatenate([sends[c][2 * c:2 * c + 2] for c in range(n)])          # chunk c = elements 2c, 2c+1
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), op
    # A NaN pins the operand order of each step: std::max(local, received) is (local < received) ? received : local,
    # false whenever either is NaN, so it returns LOCAL.  n = 4, one element per chunk; chunk c travels c+1, c+2, c+3, c.
    # NaN on the second rank of the chain: that rank keeps its NaN, the next rank keeps its own value over the NaN,
    # and the first rank's value -- however large -- is never seen again.
    nan, big = f(np.nan), f(1e30)
    sends = [np.zeros(4, f) for _ in range(4)]
    for c in range(4):
        sends[(c + 1) % 4][c] = big            # first on the chain: lost behind the NaN
        sends[(c + 2) % 4][c] = nan            # second: max(NaN, big) = NaN
        sends[(c + 3) % 4][c] = f(2.0)         # third: max(2, NaN) = 2
        sends[c][c] = f(1.0)                   # last: max(1, 2) = 2
    got = O.bootstrap_allreduce(sends, F32, MAX)[0]
    assert np.array_equal(got, np.full(4, 2.0, f))
    got = O.bootstrap_allreduce(sends, F32, MIN)[0]          # min(2, NaN) = 2, min(1, 2) = 1
    assert np.array_equal(got, np.full(4, 1.0, f))
    for c in range(4):                                        # NaN on the LAST rank of the chain is the result
        sends[(c + 2) % 4][c], sends[c][c] = f(3.0), nan
    got = O.bootstrap_allreduce(sends, F32, MAX)[0]
    assert np.isnan(got).all()
    # closed form of the reference's collective tests holds on this path too
    i = np.arange(1001)
    sends = [(r * 1000 + i % 10).astype(f) for r in range(8)]
    assert np.array_equal(O.bootstrap_allreduce(sends, F32, SUM)[5], (28 * 1000 + 8 * (i % 10)).astype(f))


# ---- avg: this path's own definition (parity unpinned by the reference) -----------------------
def test_avg_is_the_sum_divided_once():
    """Sum as defined above, then one division by k before the final rounding:
    IEEE division for floating types, C division (toward zero) of the wrapped sum
    for signed integers, unsigned division otherwise.  Checked against numpy and
    Python integers; chains of two-input passes refuse it."""
    AVG = 4
    rng = np.random.default_rng(44)
    for k in (1, 2, 3, 7, 8):
        f = [rng.uniform(-1, 1, 5000).astype(np.float32) for _ in range(k)]
        acc = f[0].copy()
        for x in f[1:]:
            acc = acc + x
        assert np.array_equal(O.reduce_copy(f, F32, AVG), acc / np.float32(k))
        d = [rng.uniform(-1, 1, 5000) for _ in range(k)]
        acc = d[0].copy()
        for x in d[1:]:
            acc = acc + x
        assert np.array_equal(O.reduce_copy(d, 8, AVG), acc / float(k))
        # 16-bit: fp32 sum / k rounded once
        h = [rng.normal(0, 1, 5000).astype(np.float16) for _ in range(k)]
        acc = h[0].astype(np.float32)
        for x in h[1:]:
            acc = acc + x.astype(np.float32)
        assert np.array_equal(O.reduce_copy([x.view(np.uint16) for x in h], F16, AVG),
                              (acc / np.float32(k)).astype(np.float16).view(np.uint16))
        b = [(rng.normal(0, 1, 5000).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16) for _ in range(k)]
        acc = (b[0].astype(np.uint32) << 16).view(np.float32)
        for x in b[1:]:
            acc = acc + (x.astype(np.uint32) << 16).view(np.float32)
        want = np.array([O.lib.oracle_f32_to_bf16(float(v)) for v in (acc / np.float32(k))], np.uint16)
        assert np.array_equal(O.reduce_copy(b, BF16, AVG), want)
        for dtype, t in ((0, np.int8), (1, np.uint8), (I32, np.int32), (3, np.uint32), (4, np.int64), (5, np.uint64)):
            t = np.dtype(t)
            lo, hi, bits = int(np.iinfo(t).min), int(np.iinfo(t).max), 8 * t.itemsize
            ins = [rng.integers(lo, hi, 300, dtype=t, endpoint=True) for _ in range(k)]
            want = []
            for col in zip(*[a.tolist() for a in ins]):
                tot = sum(col) % (1 << bits)
                if lo < 0 and tot >= 1 << (bits - 1):
                    tot -= 1 << bits
                want.append(int(tot / k) if abs(tot) < 2**52 else (abs(tot) // k) * (1 if tot >= 0 else -1))
            assert O.reduce_copy(ins, dtype, AVG).tolist() == want, (dtype, k)
    with pytest.raises(ValueError):
        O.host_ring_passes([np.zeros(4, np.float32)] * 3, F32, AVG)
    with pytest.raises(ValueError):
        O.ring_allreduce([np.zeros(4, np.float32)] * 3, F32, AVG)
    with pytest.raises(ValueError):
        O.tree_reduce([np.zeros(4, np.float32)] * 3, 0, F32, AVG)


# ---- partition arithmetic ------------------------------------------------------------------
def test_split_tiles_exactly_and_is_balanced():
    for total, parts in itertools.product([0, 1, 5, 7, 8, 9, 64, 1000, 33554432, 33554433], [1, 2, 3, 7, 8, 16]):
        pos, cnts = 0, []
        for i in range(parts):
            c, o = O.split(total, parts, i)
            assert o == pos
            pos += c
            cnts.append(c)
        assert pos == total
        assert max(cnts) - min(cnts) <= 1
        assert cnts == sorted(cnts, reverse=True)      # the first `rem` parts get the extra element
        # direct re-evaluation of the quoted formula (uni_runner_impl.cc:100-131)
        base, rem = divmod(total, parts)
        assert cnts == [base + (1 if i < rem else 0) for i in range(parts)]


def test_nredslices_reference_cases():
    # BASELINE.json configs[1]: 33,554,432 elements, 8 ranks, 8 slices, 262,144-element pieces -> 2
    assert O.lib.oracle_nredslices(33554432, 8, 8, 0, 262144) == 2
    assert O.lib.oracle_nredslices(33554432, 8, 1, 0, 65536) == 64
    assert O.lib.oracle_nredslices(0, 8, 1, 0, 65536) == 1
    assert O.lib.oracle_nredslices(100, 8, 1, 0, 0) == 1
    assert O.lib.oracle_nredslices(100, 8, 1, 5, 65536) == 5
    assert O.lib.oracle_nredslices(5, 8, 1, 0, 65536) == 1
    assert O.lib.oracle_nredslices(65536 * 8 + 1, 8, 1, 0, 65536) == 2     # float ceil just above 1


@pytest.mark.parametrize("count,n,S,R", [(33554432, 8, 8, 2), (1000003, 8, 3, 2), (17, 4, 2, 3), (5, 8, 1, 1),
                                          (64, 2, 1, 1), (12345, 3, 4, 5)])
def test_ring_allreduce_plan_covers_every_foreign_chunk_once(count, n, S, R):
    for rank in range(n):
        nodes = O.plan_ring_ar(count, n, rank, S, R)
        assert len(nodes) == S * (n - 1) * R
        covered = np.zeros(count, np.int32)
        for nd in nodes:
            assert nd.in1_off == nd.in2_off == nd.out_off and (nd.in1_buf, nd.in2_buf, nd.out_buf) == (1, 0, 1)
            covered[nd.out_off:nd.out_off + nd.count] += 1
        # every chunk except the one this rank sends first, (rank)%n, is reduced here exactly once
        c_own, o_own = O.split(count, n, rank)
        expect = np.ones(count, np.int32)
        expect[o_own:o_own + c_own] = 0
        assert np.array_equal(covered, expect)
        # step i reduces chunk (rank-i-1)%n
        for nd in nodes:
            c, o = O.split(count, n, (rank - nd.step - 1) % n)
            assert o <= nd.out_off and nd.out_off + nd.count <= o + c


@pytest.mark.parametrize("rc,n,S,R", [(4194304, 8, 8, 2), (1001, 4, 3, 2), (7, 3, 2, 2), (1, 2, 1, 1)])
def test_ring_reduce_scatter_plan(rc, n, S, R):
    for rank in range(n):
        nodes = O.plan_ring_rs(rc, n, rank, S, R)
        last = [nd for nd in nodes if nd.step == n - 2]
        out = np.zeros(rc, np.int32)
        for nd in last:                       # the last step tiles recvbuff exactly (uni_runner_impl.cc:1204-1216)
            assert nd.out_buf == 1
            out[nd.out_off:nd.out_off + nd.count] += 1
            assert nd.in1_off == rank * rc + nd.out_off          # chunk (rank-n)%n == rank
        assert (out == 1).all()
        for nd in nodes:
            if nd.step != n - 2:
                assert nd.out_buf == 2 and nd.out_off == nd.in1_off
                assert nd.in1_off // rc == (rank - nd.step - 2) % n or nd.count == 0


def test_locred_plan():
    nodes = O.plan_locred(1003, 4, 1, 3)
    c, o = O.split(1003, 4, 1)
    assert sum(nd.count for nd in nodes) == c and nodes[0].out_off == o
    assert all(a.out_off + a.count == b.out_off for a, b in zip(nodes, nodes[1:]))


# ---- ring allreduce closed forms of the reference's collective tests ---------------------------
@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_ring_allreduce_closed_forms(n):
    count = 1000 + n
    i = np.arange(count)
    # test/unittest/runner/coll_allreduce.cpp:9-37: rank*1000 + i%10 -> n(n-1)/2*1000 + n*(i%10)
    sends = [(r * 1000 + i % 10).astype(np.float32) for r in range(n)]
    for recv in O.ring_allreduce(sends, F32, SUM):
        assert np.array_equal(recv, (n * (n - 1) // 2 * 1000 + n * (i % 10)).astype(np.float32))
    # test/unittest/kernel/coll_deviceptr_allreduce.cpp:72-73: (rank+1) -> n(n+1)/2
    sends = [np.full(count, r + 1, np.float32) for r in range(n)]
    for recv in O.ring_allreduce(sends, F32, SUM):
        assert (recv == n * (n + 1) / 2).all()
    # test/perf/host_api/test_allreduce.cpp:20-32: (i%10) * 2^(rank%30), exact in fp32
    sends = [((i % 10) * 2.0 ** (r % 30)).astype(np.float32) for r in range(n)]
    want = sum(s.astype(np.float64) for s in sends).astype(np.float32)
    for recv in O.ring_allreduce(sends, F32, SUM):
        assert np.array_equal(recv, want)
    # the intra-node kernel's own checks: (rank+1) -> n(n+1)/2 through the k-way fold in rank order
    # (test/unittest/device_api/test_device_api_intra.cpp:363-389, test/perf/device_api/test_allreduce_intranode.cpp:196-211)
    assert (O.reduce_copy([np.full(count, r + 1, np.float32) for r in range(n)], F32, SUM) == n * (n + 1) / 2).all()
    # fixture pattern (i%10) + seed with seed = rank, compared as verifyBuffer does (test/fixtures/test_utils.hpp:11-34)
    got = O.reduce_copy([((i % 10) + r).astype(np.float32) for r in range(n)], F32, SUM)
    want = (n * (i % 10) + n * (n - 1) // 2).astype(np.float64)
    assert (np.abs(got - want) / np.maximum(np.abs(want), 1e-10)).max() <= 1e-5 and np.array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_reference_data_file_identical_inputs(n):
    """test/unittest/main.cpp:15-58: every rank sends i % 10, the all-reduced sum
    divided by the rank count is the input again; the suite's data file
    (test/unittest/baseline_result.txt, 1000 values) is that pattern."""
    import os
    fixture = np.loadtxt(os.path.join(os.path.dirname(__file__), "golden", "reference_baseline_result.txt"),
                         dtype=np.float32)
    assert fixture.shape == (1000,)
    sends = [fixture.copy() for _ in range(n)]
    for recv in O.ring_allreduce(sends, F32, SUM):
        assert np.array_equal(recv / n, fixture)
    assert np.array_equal(O.reduce_copy(sends, F32, SUM) / n, fixture)
    assert np.array_equal(O.reduce_copy(sends, F32, 4), fixture)      # 4 = flagcxAvg
    if n > 1:
        assert np.array_equal(O.bootstrap_allreduce(sends, F32, SUM)[0] / n, fixture)


def test_ring_allreduce_order_is_the_rotated_left_fold():
    """Chunk c of a ring allreduce equals the k-way fold starting at rank c."""
    rng = np.random.default_rng(6)
    n, count = 5, 103
    sends = [_rand_f32(rng, count) for _ in range(n)]
    recvs = O.ring_allreduce(sends, F32, SUM)
    for c in range(n):
        cnt, off = O.split(count, n, c)
        want = O.reduce_copy([s[off:off + cnt] for s in sends], F32, SUM, first=c)
        for r in range(n):
            assert np.array_equal(recvs[r][off:off + cnt].view(np.uint32), want.view(np.uint32))


# ---- binomial tree reduce (uni_runner_impl.cc:1266-1557) -----------------------------------------
def test_tree_reduce_associations_derived_by_hand():
    """Receive steps: root ceil(log2 n); others ctz(a) clipped to a + 2^i < n.  Each
    hop computes received + own.  Values chosen so that every association differs."""
    f = np.float32
    steps = lambda n: [O.lib.oracle_tree_steps(a, n) for a in range(n)]
    assert steps(8) == [3, 0, 1, 0, 2, 0, 1, 0]
    assert steps(5) == [3, 0, 1, 0, 0]
    assert steps(6) == [3, 0, 1, 0, 1, 0]
    assert steps(3) == [2, 0, 0] and steps(2) == [1, 0] and steps(7) == [3, 0, 1, 0, 2, 0, 0]
    rng = np.random.default_rng(11)
    x = [(rng.standard_normal(4000) * 10.0 ** rng.integers(-6, 7, 4000)).astype(f) for _ in range(8)]
    add = lambda a, b: (a + b).astype(f)
    want = {
        3: add(x[2], add(x[1], x[0])),
        5: add(x[4], add(add(x[3], x[2]), add(x[1], x[0]))),
        6: add(add(x[5], x[4]), add(add(x[3], x[2]), add(x[1], x[0]))),
        8: add(add(add(x[7], x[6]), add(x[5], x[4])), add(add(x[3], x[2]), add(x[1], x[0]))),
    }
    for n, w in want.items():
        got = O.tree_reduce(x[:n], 0, F32, SUM)
        assert np.array_equal(got.view(np.uint32), w.view(np.uint32)), n
        # a different order would not have matched (n = 3 is the left fold up to commutativity)
        if n > 3:
            assert not np.array_equal(got.view(np.uint32), O.reduce_copy(x[:n], F32, SUM).view(np.uint32)), n
    # root r renumbers ranks: tree rank a is rank (a + r) % n
    got = O.tree_reduce(x[:5], 2, F32, SUM)
    y = [x[(a + 2) % 5] for a in range(5)]
    assert np.array_equal(got, add(y[4], add(add(y[3], y[2]), add(y[1], y[0]))))


@pytest.mark.parametrize("n", [1, 2, 3, 4, 7, 8])
def test_tree_reduce_closed_forms(n):
    # test/unittest/runner/coll_reduce.cpp uses the allreduce pattern at the root
    count = 999
    i = np.arange(count)
    sends = [(r * 1000 + i % 10).astype(np.float32) for r in range(n)]
    for root in {0, n - 1}:
        assert np.array_equal(O.tree_reduce(sends, root, F32, SUM), (n * (n - 1) // 2 * 1000 + n * (i % 10)).astype(np.float32))
    ints = [np.full(count, r + 1, np.int32) for r in range(n)]
    assert (O.tree_reduce(ints, 0, I32, MAX) == n).all() and (O.tree_reduce(ints, 0, I32, MIN) == 1).all()


# ---- alltoallv pack / unpack ----------------------------------------------------------------------
def test_pack_unpack_round_trip_and_layout():
    rng = np.random.default_rng(8)
    counts = [5, 0, 17, 1, 1024, 3, 0, 77]
    gaps = rng.integers(0, 9, len(counts))
    order = rng.permutation(len(counts))
    displs, pos = [0] * len(counts), 0
    for i in order:                         # non-overlapping segments in shuffled order with gaps
        pos += int(gaps[i])
        displs[i] = pos
        pos += counts[i]
    send = rng.integers(0, 2**32, pos + 5, dtype=np.uint64).astype(np.uint32)
    packed = O.pack(send, counts, displs)
    slot = 0
    for c, d in zip(counts, displs):        # closed form: packed[slot_i + j] = send[displ_i + j]
        assert np.array_equal(packed[slot:slot + c], send[d:d + c])
        slot += c
    recv = np.full_like(send, 0xDEADBEEF)
    O.unpack(recv, packed, counts, displs)
    touched = np.zeros(send.size, bool)
    for c, d in zip(counts, displs):
        touched[d:d + c] = True
    assert np.array_equal(recv[touched], send[touched])
    assert (recv[~touched] == 0xDEADBEEF).all()


# ---- reduce trigger bit layout: flagcx_kernel_core.h:146-162 ---------------------------------------
def test_trigger_layout_constants():
    v = O.trigger_encode(0x1111, 0x2222, 0x3333, 0xABCDEF01, 0x1234, 9, 3, 1)
    assert v[:3] == [0x1111, 0x2222, 0x3333]
    w = v[3]
    assert w & 0xffffffff == 0xABCDEF01            # count: offset 0, 32 bits
    assert (w >> 32) & 0xffff == 0x1234            # nthreads: offset 32, 16 bits
    assert (w >> 48) & 0xf == 9                    # datatype: offset 48, 4 bits
    assert (w >> 52) & 0xf == 3                    # redop: offset 52, 4 bits
    assert (w >> 56) & 0x3 == 1                    # state: offset 56, 2 bits
    assert w >> 58 == 0
    # fields are masked, not allowed to spill into their neighbours
    v = O.trigger_encode(0, 0, 0, 2**40 - 1, 2**20 - 1, 31, 31, 7)
    assert v[3] == 0xffffffff | (0xffff << 32) | (0xf << 48) | (0xf << 52) | (0x3 << 56)


# --- the reference device kernel's own 16-bit arithmetic (custom_allreduce.cu:326-361) -----------------------------

BF = lambda *v: [np.array([x], np.uint16) for x in v]            # one element per input, given as bit patterns


def test_element_fold_rounds_after_every_addition():
    """bf16 has 8 significant bits: 256 + 1 = 257 is a tie between 256 and 258
    and goes to the even one, 256, and so does the next + 1; rounding once gives
    258.  fp16 has 11: the same with 2048 and 2050.  Worked out by hand."""
    b256, b1, b258, b2 = 0x4380, 0x3F80, 0x4381, 0x4000
    assert O.reduce_copy_elem(BF(b256, b1, b1), BF16, SUM)[0] == b256
    assert O.reduce_copy(BF(b256, b1, b1), BF16, SUM)[0] == b258          # the default arithmetic
    h2048, h1, h2050 = 0x6800, 0x3C00, 0x6801
    assert O.reduce_copy_elem(BF(h2048, h1, h1), F16, SUM)[0] == h2048
    assert O.reduce_copy(BF(h2048, h1, h1), F16, SUM)[0] == h2050
    # the steps run left to right from `first`: 1 + 1 = 2, 2 + 256 = 258 exactly; 256 + 1 first loses both ones
    assert O.reduce_copy_elem(BF(b1, b1, b256), BF16, SUM)[0] == b258
    assert O.reduce_copy_elem(BF(b256, b1, b1), BF16, SUM, first=1)[0] == b258
    assert O.reduce_copy_elem(BF(b1, b256, b1), BF16, SUM)[0] == b256
    assert O.reduce_copy_elem(BF(b1, b1), BF16, SUM)[0] == b2


@pytest.mark.parametrize("dtype", [BF16, F16])
def test_element_fold_max_min_hand_on_the_later_operand(dtype):
    """a > b ? a : b with a the accumulator (custom_allreduce.cu:329-331): a
    tie or an unordered pair yields b.  Every case below is that rule applied by
    hand; the host rule (std::max, the default here) gives the other answer
    wherever the comment says so."""
    if dtype == BF16:
        one, two, three, five, pz, nz, nan = 0x3F80, 0x4000, 0x4040, 0x40A0, 0x0000, 0x8000, 0x7FC0
    else:
        one, two, three, five, pz, nz, nan = 0x3C00, 0x4000, 0x4200, 0x4500, 0x0000, 0x8000, 0x7E00
    e = lambda op, *v: int(O.reduce_copy_elem(BF(*v), dtype, op)[0])
    d = lambda op, *v: int(O.reduce_copy(BF(*v), dtype, op)[0])
    assert e(MAX, pz, nz) == nz and d(MAX, pz, nz) == pz          # +0 > -0 is false: the later one
    assert e(MAX, nz, pz) == pz and d(MAX, nz, pz) == nz
    assert e(MIN, nz, pz) == pz and e(MIN, pz, nz) == nz
    assert e(MAX, one, nan, pz) == pz and d(MAX, one, nan, pz) == one      # 1 -> NaN -> 0: the NaN resets the fold
    assert e(MAX, nan, three, five) == five and d(MAX, nan, three, five) == nan
    assert e(MAX, one, two, nan) == nan and d(MAX, one, two, nan) == two
    assert e(MIN, one, nan, five) == five and e(MIN, five, three, nan) == nan
    assert e(MAX, one, five, three) == five and e(MIN, five, one, three) == one     # ordered values: plain max / min
    with pytest.raises(ValueError):
        O.reduce_copy_elem(BF(one, two), dtype, PROD)
    with pytest.raises(ValueError):
        O.reduce_copy_elem([np.ones(3, np.float32)] * 2, F32, SUM)


@pytest.mark.parametrize("dtype", [BF16, F16])
def test_element_fold_steps_are_single_correctly_rounded_additions(dtype):
    """Two inputs: one addition, one rounding -- the pinned default oracle's
    answer.  More inputs, fp16: every step is numpy's float16 addition."""
    rng = np.random.default_rng(7)
    n = 200000
    if dtype == F16:
        ins = [(rng.standard_normal(n) * 10 ** rng.uniform(-4, 4, n)).astype(np.float16).view(np.uint16) for _ in range(5)]
    else:
        ins = [((rng.standard_normal(n) * 10 ** rng.uniform(-6, 6, n)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
               for _ in range(5)]
    assert np.array_equal(O.reduce_copy_elem(ins[:2], dtype, SUM), O.reduce_copy(ins[:2], dtype, SUM))
    if dtype == F16:
        with np.errstate(over="ignore", invalid="ignore"):
            acc = ins[0].view(np.float16)
            for x in ins[1:]:
                acc = acc + x.view(np.float16)
        got = O.reduce_copy_elem(ins, dtype, SUM).view(np.float16)
        same = (got.view(np.uint16) == acc.view(np.uint16)) | (np.isnan(got) & np.isnan(acc))
        assert same.all()
    else:   # bf16: a second, arithmetic rounding of each exact step (float64 holds the sum of two bf16 values exactly)
        acc = (ins[0].astype(np.uint32) << 16).view(np.float32)
        for x in ins[1:]:
            exact = acc.astype(np.float64) + (x.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
            m, ex = np.frexp(exact)                            # exact = m * 2**ex, 0.5 <= |m| < 1: keep 8 significant bits
            acc = np.ldexp(np.rint(m * 256.0), ex - 8).astype(np.float32)      # rint is round-half-even
        got = (O.reduce_copy_elem(ins, dtype, SUM).astype(np.uint32) << 16).view(np.float32)
        assert np.array_equal(got, acc)
