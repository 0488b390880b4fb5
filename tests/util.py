"""Shared helpers for the parity tests."""
import numpy as np

from flagcx_amd import _native as N
from flagcx_amd import kernels as K

DTYPES = {"fp32": N.DT_FP32, "int32": N.DT_INT32, "bf16": N.DT_BF16, "fp16": N.DT_FP16,
          "uint32": N.DT_UINT32, "int8": N.DT_INT8, "uint8": N.DT_UINT8, "int64": N.DT_INT64, "uint64": N.DT_UINT64,
          "fp64": N.DT_FP64}
OPS = {"sum": N.OP_SUM, "prod": N.OP_PROD, "max": N.OP_MAX, "min": N.OP_MIN, "avg": N.OP_AVG}


def seeded_inputs(dtype, k, n, seed, dist=None):
    """k host arrays of n elements in the distribution BASELINE.json's configs name
    for the type: fp32 uniform[-1,1), 16-bit N(0,1), int32 uniform[-2^20,2^20].
    The other host types of the reference (8/64-bit and unsigned integers over
    their whole range so that sums and products wrap, fp64 uniform[-1,1)) come
    from numpy's seeded generator."""
    out = []
    for p in range(k):
        if dtype in (N.DT_INT8, N.DT_UINT8, N.DT_UINT32, N.DT_INT64, N.DT_UINT64):
            t = np.dtype(N.NP_DTYPE[dtype])
            rng = np.random.default_rng([seed, p, dtype])
            out.append(rng.integers(np.iinfo(t).min, np.iinfo(t).max, n, dtype=t, endpoint=True))
        elif dtype == N.DT_FP64:
            out.append(np.random.default_rng([seed, p, dtype]).uniform(-1.0, 1.0, n))
        elif dtype == N.DT_FP32:
            out.append(K.synth(n, dtype, K.SYNTH_UNIFORM, -1.0, 1.0, seed, p))
        elif dtype == N.DT_INT32:
            out.append(K.synth(n, dtype, K.SYNTH_UNIFORM_INT, -(1 << 20), 1 << 20, seed, p))
        else:
            mean, std = dist or (0.0, 1.0)
            out.append(K.synth(n, dtype, K.SYNTH_NORMAL, mean, std, seed, p))
    return out


def is_nan16(bits, dtype):
    bits = bits.astype(np.uint32)
    if dtype == N.DT_BF16:
        return (bits & 0x7fff) > 0x7f80
    return (bits & 0x7fff) > 0x7c00


def ordered16(bits):
    """Map 16-bit sign-magnitude float patterns to a monotone integer line."""
    b = bits.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7fff), b & 0x7fff)


def assert_parity(got, want, dtype, op, what=""):
    """Bit-exact for fp32 / fp64 / integers / every max-min; for 16-bit sum, prod
    and avg the stated tolerance is 1 ulp of the output type, NaN matching NaN."""
    assert got.shape == want.shape
    if dtype in (N.DT_BF16, N.DT_FP16) and op in (N.OP_SUM, N.OP_PROD, N.OP_AVG):
        gn, wn = is_nan16(got, dtype), is_nan16(want, dtype)
        assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
        d = np.abs(ordered16(got)[~gn] - ordered16(want)[~wn])
        assert d.size == 0 or d.max() <= 1, f"{what}: max ulp distance {d.max()}"
        return int((d != 0).sum())
    g, w = got.view(np.uint8), want.view(np.uint8)
    if not np.array_equal(g, w):
        bad = np.nonzero(got.view(_uint(got)) != want.view(_uint(want)))[0]
        raise AssertionError(f"{what}: {bad.size} mismatches, first at {bad[0]}: "
                             f"got {got[bad[0]]!r} want {want[bad[0]]!r}")
    return 0


def _uint(a):
    return {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.itemsize]


class DevBufs:
    """Device allocations that are freed together."""

    def __init__(self, dev):
        self.dev, self.ptrs = dev, []

    def alloc(self, nbytes):
        p = self.dev.malloc(nbytes)
        self.ptrs.append(p)
        return p

    def put(self, host, pad_before=0, pad_after=0):
        """Upload `host` at byte offset pad_before inside a fresh allocation."""
        base = self.alloc(pad_before + host.nbytes + pad_after + 64)
        self.dev.upload(base + pad_before, host)
        return base + pad_before

    def close(self):
        for p in self.ptrs:
            self.dev.free(p)
        self.ptrs = []

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()
