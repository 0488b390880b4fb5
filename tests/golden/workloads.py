"""The configurations of BASELINE.json as data: shapes, seeds, distributions.  Shared by
the fixture generator, the parity tests and nothing else."""
import hashlib

import numpy as np

from flagcx_amd import _native as N
from flagcx_amd import kernels as K

# name -> (dtype, k, elements per input, distribution, seed)
CFG1 = dict(dtype=N.DT_FP32, k=2, n=16_777_216, dist=(K.SYNTH_UNIFORM, -1.0, 1.0), seed=0)
CFG2 = dict(dtype=N.DT_BF16, k=8, n=33_554_432, dist=(K.SYNTH_NORMAL, 0.0, 1.0), seed=1,
            nslices=8, redslice_elems=262_144)        # 512 KiB pieces
CFG3 = dict(k=4, seed=2, min_bytes=1 << 10, max_bytes=1 << 30,
            dists={N.DT_FP16: (K.SYNTH_NORMAL, 0.0, 1.0), N.DT_FP32: (K.SYNTH_UNIFORM, -1.0, 1.0),
                   N.DT_INT32: (K.SYNTH_UNIFORM_INT, -(1 << 20), 1 << 20)})
CFG4 = dict(dtype=N.DT_FP32, npeers=8, seed=3, min_count=1, max_count=4_194_304)
CFG5 = dict(dtype=N.DT_BF16, k=8, n=268_435_456, dist=(K.SYNTH_NORMAL, 0.0, 0.02), seed=4)

OPS = {"sum": N.OP_SUM, "prod": N.OP_PROD, "max": N.OP_MAX, "min": N.OP_MIN}
DTYPE_NAMES = {N.DT_FP32: "fp32", N.DT_FP16: "fp16", N.DT_BF16: "bf16", N.DT_INT32: "int32"}


def inputs(dtype, k, n, dist, seed, threads=8, first_stream=0):
    kind, a, b = dist
    return [K.synth(n, dtype, kind, a, b, seed, first_stream + p, threads) for p in range(k)]


def cfg3_inputs(dtype, n, threads=8):
    """cfg3 gives no per-case seed: inputs of every size are prefixes of one
    stream per (dtype, input), seed 2, stream = 16*dtype + input."""
    return inputs(dtype, CFG3["k"], n, CFG3["dists"][dtype], CFG3["seed"], threads, first_stream=16 * dtype)


ALL_OPS = dict(OPS, avg=N.OP_AVG)
ALL_DTYPES = {"int8": N.DT_INT8, "uint8": N.DT_UINT8, "int32": N.DT_INT32, "uint32": N.DT_UINT32, "int64": N.DT_INT64,
              "uint64": N.DT_UINT64, "fp16": N.DT_FP16, "fp32": N.DT_FP32, "fp64": N.DT_FP64, "bf16": N.DT_BF16}


def matrix_inputs(dtype, k=3, n=4099, seed=5):
    """Small seeded inputs for every element type: the synthetic generator for
    the types it knows, numpy's PCG64 over the whole integer range otherwise."""
    if dtype in (N.DT_FP32, N.DT_FP64):
        return inputs(dtype, k, n, (K.SYNTH_UNIFORM, -1.0, 1.0), seed, 1)
    if dtype in (N.DT_FP16, N.DT_BF16):
        return inputs(dtype, k, n, (K.SYNTH_NORMAL, 0.0, 1.0), seed, 1)
    if dtype == N.DT_INT32:
        return inputs(dtype, k, n, (K.SYNTH_UNIFORM_INT, -(1 << 20), 1 << 20), seed, 1)
    t = np.dtype(N.NP_DTYPE[dtype])
    return [np.random.Generator(np.random.PCG64([seed, p, dtype])).integers(np.iinfo(t).min, np.iinfo(t).max, n, dtype=t,
                                                                            endpoint=True) for p in range(k)]


def cfg4_layout():
    """Per-peer counts log-uniform in [1, 4194304] from seed 3 and random
    non-overlapping displacements (shuffled segment order, gaps of 0..63
    elements) for the send side and, independently, the receive side."""
    u = K.synth(64, N.DT_FP64, K.SYNTH_UNIFORM, 0.0, 1.0, CFG4["seed"], 100)
    npeers = CFG4["npeers"]
    lo, hi = np.log(CFG4["min_count"]), np.log(CFG4["max_count"])
    counts = [int(min(CFG4["max_count"], max(CFG4["min_count"], np.floor(np.exp(lo + x * (hi - lo))))))
              for x in u[:npeers]]

    def layout(us):
        order = np.argsort(us[:npeers], kind="stable")
        gaps = (us[npeers:2 * npeers] * 64).astype(np.int64)
        displs, pos = [0] * npeers, 0
        for j, i in enumerate(order):
            pos += int(gaps[j])
            displs[int(i)] = pos
            pos += counts[int(i)]
        return displs, pos + 17

    sdispls, slen = layout(u[8:24])
    rdispls, rlen = layout(u[24:40])
    return counts, sdispls, slen, rdispls, rlen


def digest(arr):
    a = np.ascontiguousarray(arr)
    return hashlib.sha256(a.view(np.uint8)).hexdigest()


def probe(arr, m=8):
    """A few raw words from fixed positions, for a readable diff when a digest fails."""
    a = np.ascontiguousarray(arr)
    idx = [0, 1, a.size // 3, a.size // 2, a.size - 1][:m]
    w = a.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.itemsize])
    return [int(w[i]) for i in idx if a.size]
