"""Run by tests/test_gpu_policy.py in a process of its own, once per cache
policy: the policy is read from the environment once per process
(FX_CACHE_POLICY, FX_TEMPORAL_MAX_BYTES), and every flavour of load and store
the kernels carry must give the oracle's bits -- direct launches, slice batches,
multi-output launches and a plan, aligned and element-aligned inputs, sizes on
both sides of the striping and small-launch thresholds."""
import os
import sys

import numpy as np

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from flagcx_amd.adaptor import Device
from oracle import fx_oracle as O
from tests.util import DevBufs, assert_parity, seeded_inputs


def main():
    dev = Device(0)
    checked = 0
    for dname, dtype in (("bf16", N.DT_BF16), ("fp32", N.DT_FP32), ("int32", N.DT_INT32)):
        es = N.DTYPE_SIZE[dtype]
        for k in (1, 2, 3, 8):
            for n in (1000 + k, 300_007, (3 << 20) + 5):
                op = N.OP_SUM if k > 1 else N.OP_MAX
                ins = seeded_inputs(dtype, k, n, seed=7 * k + 1)
                want = O.reduce_copy(ins, dtype, op)
                with DevBufs(dev) as b:
                    # every other input one element off the output's 16-byte grid
                    dins = [b.put(a, pad_before=es * (p % 2)) for p, a in enumerate(ins)]
                    dout = b.alloc(n * es + 64)
                    N.check(K.reduce_copy(dout, dins, n, dtype, op), "fx_reduce_copy")
                    dev.sync()
                    assert_parity(dev.to_host(dout, n, N.NP_DTYPE[dtype]), want, dtype, op, f"direct {dname} k={k} n={n}")
                    # the same as three ragged slices of one batch, then as a plan
                    cuts = [0, n // 3 + 1, 2 * n // 3 - 1, n]
                    douts = [b.alloc(n * es + 64) for _ in range(2)]
                    for d in douts:
                        dev.memset(d, 0x5a, n * es + 64)
                    descs = [[([p + cuts[i] * es for p in dins], d + cuts[i] * es, cuts[i + 1] - cuts[i]) for i in range(3)]
                             for d in douts]
                    N.check(K.reduce_slices(descs[0], k, dtype, op), "fx_reduce_slices")
                    plan = K.Plan(descs[1], k, dtype, op)
                    N.check(plan.launch(), "fx_plan_launch")
                    dev.sync()
                    plan.destroy()
                    for d, what in zip(douts, ("slices", "plan")):
                        assert_parity(dev.to_host(d, n, N.NP_DTYPE[dtype]), want, dtype, op, f"{what} {dname} k={k} n={n}")
                    # one read, three stores
                    dm = [b.alloc(n * es + 64) for _ in range(3)]
                    N.check(K.reduce_bcast_slices([(dins, dm, n)], k, 3, dtype, op), "fx_reduce_bcast_slices")
                    dev.sync()
                    for d in dm:
                        assert_parity(dev.to_host(d, n, N.NP_DTYPE[dtype]), want, dtype, op, f"bcast {dname} k={k} n={n}")
                    checked += 6
    # copies: a batch that reads one source several times, and an off-phase source (grouped columns)
    src = np.random.default_rng(3).integers(0, 256, (5 << 20) + 3, dtype=np.uint8)
    with DevBufs(dev) as b:
        dsrc = b.put(src, pad_before=4)
        outs = [b.alloc(src.size + 64) for _ in range(4)]
        N.check(K.copy_slices([(dsrc, o, src.size) for o in outs]), "fx_copy_slices")
        dev.sync()
        for o in outs:
            assert np.array_equal(dev.to_host(o, src.size, np.uint8), src)
        checked += 4
    print(f"policy client ok: {checked} results under FX_CACHE_POLICY={os.environ.get('FX_CACHE_POLICY')} "
          f"FX_TEMPORAL_MAX_BYTES={os.environ.get('FX_TEMPORAL_MAX_BYTES')}")


if __name__ == "__main__":
    sys.exit(main())
