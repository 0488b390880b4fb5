"""GPU parity of the one-launch tree and keep-local associations
(fx_reduce_ordered) against the CPU oracle's step-by-step restatements of the
reference's binomial-tree reduce and host ring, and of the reference-named
consumer launcher driven by a stand-in for the reference's scheduler."""
import os
import subprocess

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from oracle import fx_oracle as O
from tests.util import DTYPES, DevBufs, seeded_inputs

pytestmark = pytest.mark.gpu

NAN16 = {"bf16": 0x7fc0, "fp16": 0x7e00}


def _with_specials(ins, dname, rng):
    """NaN (both signs) and zeros of both signs at scattered places of every input."""
    n = ins[0].size
    for p, a in enumerate(ins):
        idx = rng.choice(n, size=64, replace=False)
        if dname in NAN16:
            a[idx[:16]] = NAN16[dname]
            a[idx[16:32]] = NAN16[dname] | 0x8000
            a[idx[32:48]] = 0x0000
            a[idx[48:]] = 0x8000
        elif dname in ("fp32", "fp64"):
            a[idx[:16]] = np.nan
            a[idx[16:32]] = -np.nan
            a[idx[32:48]] = 0.0
            a[idx[48:]] = -0.0
    return ins


def _bits(a):
    return a.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.itemsize])


def _keep_local_chain(ins, dtype, op):
    """res = in[0]; res = in[j] (op) res -- the local operand of every step first
    (flagcx/service/bootstrap.cc:853-871), each step the pinned two-input oracle."""
    res = ins[0].copy()
    for j in range(1, len(ins)):
        res = O.reduce2(ins[j], res, dtype, op)
    return res


@pytest.mark.parametrize("dname", ["fp32", "bf16", "fp16", "fp64", "int32"])
@pytest.mark.parametrize("k", [2, 3, 4, 5, 6, 7, 8])
def test_tree_fold_in_one_launch_matches_the_step_by_step_tree(dev, dname, k):
    """in[a] = tree rank a; every step rounds to the element type, as the
    reference's tree does through its two-input kernel.  Two ragged slices in one
    call, three outputs each, output off the 16-byte grid."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    total = 150001
    rng = np.random.default_rng(k)
    pieces = [(3, 70001), (70011, 79990)]          # (offset, count): a gap between them, odd starts
    for op in (N.OP_SUM, N.OP_PROD, N.OP_MAX, N.OP_MIN):
        ins = seeded_inputs(dtype, k, total, seed=31 + k)
        if op in (N.OP_MAX, N.OP_MIN):
            ins = _with_specials(ins, dname, rng)
        with DevBufs(dev) as b:
            dins = [b.put(a) for a in ins]
            douts = [b.put(np.zeros(total, N.NP_DTYPE[dtype]), pad_before=es * 3) for _ in range(3)]
            descs = [([p + o * es for p in dins], [q + o * es for q in douts], c) for o, c in pieces]
            N.check(K.reduce_ordered(descs, k, 3, dtype, op, K.FOLD_TREE), "fx_reduce_ordered")
            dev.sync()
            got = [dev.to_host(q, total, N.NP_DTYPE[dtype]) for q in douts]
        want = np.zeros(total, N.NP_DTYPE[dtype])
        for o, c in pieces:
            want[o:o + c] = O.tree_reduce([a[o:o + c] for a in ins], 0, dtype, op)
        for g in got:
            assert np.array_equal(_bits(g), _bits(want)), f"tree {dname} k={k} op={op}"


@pytest.mark.parametrize("dname", ["fp32", "bf16", "fp16", "fp64"])
@pytest.mark.parametrize("k", [2, 3, 4, 5, 8])
def test_keep_local_chain_in_one_launch_matches_the_host_ring_steps(dev, dname, k):
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    total = 90007
    rng = np.random.default_rng(100 + k)
    for op in (N.OP_MAX, N.OP_MIN):
        ins = _with_specials(seeded_inputs(dtype, k, total, seed=5 + k), dname, rng)
        want = _keep_local_chain(ins, dtype, op)
        for nout in (1, k):
            with DevBufs(dev) as b:
                dins = [b.put(a) for a in ins]
                douts = [b.alloc(total * es) for _ in range(nout)]
                N.check(K.reduce_ordered([(dins, douts, total)], k, nout, dtype, op, K.FOLD_KEEP_LOCAL))
                dev.sync()
                for q in douts:
                    assert np.array_equal(_bits(dev.to_host(q, total, N.NP_DTYPE[dtype])), _bits(want)), \
                        f"keep-local {dname} k={k} op={op} nout={nout}"
    # a NaN hides what was folded before it: the chain and the input-order fold differ on these inputs
    if k >= 3:
        chain = O.reduce_copy(ins, dtype, N.OP_MIN)
        assert not np.array_equal(_bits(chain), _bits(_keep_local_chain(ins, dtype, N.OP_MIN)))


def test_keep_local_in_place_on_every_input(dev):
    """The all-reduce shape: output r aliases input r exactly."""
    dtype, k, total = N.DT_FP32, 4, 50001
    ins = _with_specials(seeded_inputs(dtype, k, total, seed=9), "fp32", np.random.default_rng(1))
    want = _keep_local_chain(ins, dtype, N.OP_MAX)
    with DevBufs(dev) as b:
        dins = [b.put(a) for a in ins]
        N.check(K.reduce_ordered([(dins, dins, total)], k, k, dtype, N.OP_MAX, K.FOLD_KEEP_LOCAL))
        dev.sync()
        for q in dins:
            assert np.array_equal(_bits(dev.to_host(q, total, np.float32)), _bits(want))


def test_orders_that_need_no_kernel_of_their_own_and_the_refused_ones(dev):
    total, k = 40001, 5
    with DevBufs(dev) as b:
        # integers: every association gives the input-order fold's bits
        ins = seeded_inputs(N.DT_INT32, k, total, seed=2)
        dins = [b.put(a) for a in ins]
        dout = b.alloc(total * 4)
        for order in (K.FOLD_TREE, K.FOLD_KEEP_LOCAL):
            for op in (N.OP_SUM, N.OP_PROD, N.OP_MAX):
                N.check(K.reduce_ordered([(dins, [dout], total)], k, 1, N.DT_INT32, op, order))
                dev.sync()
                assert np.array_equal(dev.to_host(dout, total, np.int32), O.reduce_copy(ins, N.DT_INT32, op))
        # fp32 keep-local sums: the operands of a step commute bit for bit
        fins = seeded_inputs(N.DT_FP32, k, total, seed=3)
        dfin = [b.put(a) for a in fins]
        N.check(K.reduce_ordered([(dfin, [dout], total)], k, 1, N.DT_FP32, N.OP_SUM, K.FOLD_KEEP_LOCAL))
        dev.sync()
        assert np.array_equal(_bits(dev.to_host(dout, total, np.float32)), _bits(O.reduce_copy(fins, N.DT_FP32, N.OP_SUM)))
        d = [(dfin, [dout], total)]
        assert K.reduce_ordered(d, k, 1, N.DT_FP32, N.OP_AVG, K.FOLD_TREE) == N.NOT_SUPPORTED
        assert K.reduce_ordered(d, k, 1, N.DT_BF16, N.OP_SUM, K.FOLD_KEEP_LOCAL) == N.NOT_SUPPORTED
        assert K.reduce_ordered(d, k, 1, N.DT_BF16, N.OP_SUM | 0x100, K.FOLD_TREE) == N.NOT_SUPPORTED
        assert K.reduce_ordered(d, k, 1, N.DT_FP32, N.OP_SUM, 3) == N.INVALID_ARGUMENT
        assert K.reduce_ordered(d, 9, 1, N.DT_FP32, N.OP_SUM, K.FOLD_TREE) == N.INVALID_ARGUMENT
        assert K.reduce_ordered([(dfin, [dout, dout + 4], total - 1)], k, 2, N.DT_FP32, N.OP_SUM, K.FOLD_TREE) == \
            N.INVALID_ARGUMENT          # outputs that do not share their offset within 16 bytes
        assert K.reduce_ordered([], k, 1, N.DT_FP32, N.OP_SUM, K.FOLD_TREE) == N.SUCCESS


@pytest.mark.parametrize("n,count,nslices,nred", [(4, 1_000_003, 2, 2), (8, 262_144 * 8, 8, 1), (3, 1001, 1, 1)])
def test_reference_scheduler_stand_in_runs_through_the_reference_named_launcher(tmp_path, n, count, nslices, nred):
    """flagcx_amd/lib/unirunner_client (tests/unirunner_client.cc) is what the
    reference's runUniRunner does around flagcxLaunchCollectiveKernel
    (flagcx/runner/uni_runner_impl.cc:1864-1901): launch, enqueue triggers, poll,
    set terminate, synchronise -- twice, each time with a fresh pinned ring.  The
    ring all-reduce it schedules folds chunk c in the order c, c+1, ...
    (uni_runner_impl.cc:864-878: out = received partial + own data)."""
    exe = os.path.join(N.LIB_DIR, "unirunner_client")
    sends = seeded_inputs(N.DT_FP32, n, count, seed=40 + n)
    inp, outp = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(inp, "wb") as f:
        f.write(np.array([n, count], np.uint64).tobytes())
        for s in sends:
            f.write(s.tobytes())
    env = dict(os.environ, FX_FIFO_MAX_IDLE_POLLS="20000000")      # the consumer gives up by itself should the client die
    r = subprocess.run([exe, N.PLUGIN_LIB, str(inp), str(outp), str(nslices), str(nred)], capture_output=True, text=True,
                       env=env, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "flagcxLaunchCollectiveKernel" not in r.stderr, r.stderr
    got = np.fromfile(outp, np.float32).reshape(n, count)
    want = np.empty(count, np.float32)
    for c in range(n):
        cnt, off = K.split(count, n, c)
        want[off:off + cnt] = O.reduce_copy([s[off:off + cnt] for s in sends], N.DT_FP32, N.OP_SUM, first=c)
    for r_ in range(n):
        assert np.array_equal(got[r_].view(np.uint32), want.view(np.uint32)), f"rank {r_}"
