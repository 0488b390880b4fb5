"""Seeded random parity runs: the C ABI on the GPU against the CPU oracle over
cases nobody picked by hand -- type, op, input count, length, alignment of
every buffer, in place or not, slicing, number of outputs, fold order,
algorithm, ring capacity.  Every case prints its description before it touches
the GPU, so a failure names it; the seeds are fixed, so it repeats."""
import ctypes as C

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from flagcx_amd import sim as S
from oracle import fx_oracle as O
from tests.util import DTYPES, OPS, DevBufs, assert_parity, seeded_inputs

pytestmark = pytest.mark.gpu

PAD = 0xA5


def _fresh_out(b, dev, lead_bytes, nbytes):
    base = b.alloc(lead_bytes + nbytes + 256)
    dev.memset(base, PAD, lead_bytes + nbytes + 256)
    return base + lead_bytes


def _kernel_case(dev, rng, no):
    names = list(DTYPES)
    dname = names[rng.integers(len(names))]
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    op = list(OPS.values())[rng.integers(len(OPS))]
    k = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 13]))
    n = int(rng.integers(1, 6_000_000 // es)) if rng.random() < 0.1 else int(rng.integers(1, 40000))
    if k > 8:
        n = min(n, 200000)
    mode = int(rng.integers(4))       # 0 reduce_copy, 1 slices, 2 several outputs, 3 reduce_copy in place
    if k > 8 and mode in (1, 2):
        mode = 0                      # the slice descriptors carry at most 8 inputs
    ve = 16 // es
    same = rng.random() < 0.6         # every buffer aligned alike, or each at its own offset
    o0 = int(rng.integers(0, ve * 40))
    offs = [o0 if same else int(rng.integers(0, ve * 40)) for _ in range(k)]
    first = int(rng.integers(k)) if mode in (0, 3) else 0
    seed = int(rng.integers(1 << 30))
    desc = f"case {no}: {dname} op={op} k={k} n={n} mode={mode} out+{o0} in+{offs} first={first} seed={seed}"
    print(desc, flush=True)
    ins = seeded_inputs(dtype, k, n, seed=seed)
    want = O.reduce_copy(ins, dtype, op, first=first)
    with DevBufs(dev) as b:
        dins = [b.put(a, pad_before=o * es, pad_after=64) for a, o in zip(ins, offs)]
        if mode == 3:
            outs = [dins[int(rng.integers(k))]]
            N.check(K.reduce_copy(outs[0], dins, n, dtype, op, first), desc)
        elif mode == 0:
            outs = [_fresh_out(b, dev, o0 * es, n * es)]
            N.check(K.reduce_copy(outs[0], dins, n, dtype, op, first), desc)
        elif mode == 1:
            outs = [_fresh_out(b, dev, o0 * es, n * es)]
            cuts = sorted(set(int(x) for x in rng.integers(0, n + 1, int(rng.integers(0, 6)))))
            edges = [0] + cuts + [n]
            descs = [([p + lo * es for p in dins], outs[0] + lo * es, hi - lo) for lo, hi in zip(edges[:-1], edges[1:])]
            N.check(K.reduce_slices(descs, k, dtype, op), desc)
        else:
            outs = [_fresh_out(b, dev, (o0 if rng.random() < 0.8 else int(rng.integers(0, ve * 4))) * es, n * es)
                    for _ in range(int(rng.integers(1, 9)))]
            N.check(K.reduce_bcast_slices([(dins, outs, n)], k, len(outs), dtype, op), desc)
        dev.sync()
        for d in outs:
            assert_parity(dev.to_host(d, n, N.NP_DTYPE[dtype]), want, dtype, op, desc)
            if mode != 3:
                assert (dev.to_host(d + n * es, 32, np.uint8) == PAD).all(), "wrote past the end: " + desc
                if d % 16:
                    lead = d % 16
                    assert (dev.to_host(d - lead, lead, np.uint8) == PAD).all(), "wrote before the start: " + desc


def test_kernel_layer_random_cases(dev):
    rng = np.random.default_rng(20240611)
    for no in range(3000):
        _kernel_case(dev, rng, no)


def _ordered_case(dev, rng, no):
    """fx_reduce_ordered: tree or keep-local association, any type, 2..8 inputs, one to eight outputs, the inputs
    each at their own offset, one or two slices; NaNs and signed zeros planted for max / min."""
    names = ["fp32", "fp64", "bf16", "fp16", "int32", "uint8", "int64"]
    dname = names[rng.integers(len(names))]
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    order = int(rng.choice([K.FOLD_TREE, K.FOLD_KEEP_LOCAL]))
    op = int(rng.choice([N.OP_SUM, N.OP_PROD, N.OP_MAX, N.OP_MIN]))
    k = int(rng.integers(2, 9))
    if order == K.FOLD_KEEP_LOCAL and dname in ("bf16", "fp16") and op in (N.OP_SUM, N.OP_PROD) and k >= 3:
        op = N.OP_MAX                 # the one combination the entry point refuses (no such host path)
    n = int(rng.integers(1, 3_000_000 // es)) if rng.random() < 0.1 else int(rng.integers(1, 40000))
    nout = int(rng.integers(1, 9))
    ve = 16 // es
    o0 = int(rng.integers(0, ve * 40))
    offs = [o0 if rng.random() < 0.5 else int(rng.integers(0, ve * 40)) for _ in range(k)]
    cut = int(rng.integers(0, n + 1))
    seed = int(rng.integers(1 << 30))
    desc = f"ordered case {no}: {dname} order={order} op={op} k={k} n={n} nout={nout} out+{o0} in+{offs} cut={cut} seed={seed}"
    print(desc, flush=True)
    ins = seeded_inputs(dtype, k, n, seed=seed)
    if op in (N.OP_MAX, N.OP_MIN) and dname in ("fp32", "fp64", "bf16", "fp16") and n > 64:
        for a in ins:
            idx = rng.choice(n, size=min(32, n), replace=False)
            if dname in ("bf16", "fp16"):
                nan = 0x7fc0 if dname == "bf16" else 0x7e00
                a[idx[:8]], a[idx[8:16]], a[idx[16:24]], a[idx[24:]] = nan, nan | 0x8000, 0x0000, 0x8000
            else:
                a[idx[:8]], a[idx[8:16]], a[idx[16:24]], a[idx[24:]] = np.nan, -np.nan, 0.0, -0.0
    if order == K.FOLD_TREE:
        want = O.tree_reduce(ins, 0, dtype, op)
    else:
        want = ins[0].copy()
        for j in range(1, k):
            want = O.reduce2(ins[j], want, dtype, op)
    with DevBufs(dev) as b:
        dins = [b.put(a, pad_before=o * es, pad_after=64) for a, o in zip(ins, offs)]
        outs = [_fresh_out(b, dev, o0 * es, n * es) for _ in range(nout)]
        descs = [([p + lo * es for p in dins], [q + lo * es for q in outs], hi - lo) for lo, hi in ((0, cut), (cut, n))]
        N.check(K.reduce_ordered(descs, k, nout, dtype, op, order), desc)
        dev.sync()
        for d in outs:
            got = dev.to_host(d, n, N.NP_DTYPE[dtype])
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), desc
            assert (dev.to_host(d + n * es, 32, np.uint8) == PAD).all(), "wrote past the end: " + desc
            if d % 16:
                lead = d % 16
                assert (dev.to_host(d - lead, lead, np.uint8) == PAD).all(), "wrote before the start: " + desc


def test_ordered_folds_random_cases(dev):
    rng = np.random.default_rng(20241125)
    for no in range(1200):
        _ordered_case(dev, rng, no)


def _collective_case(dev, stream, rng, no):
    names = ["fp32", "int32", "fp64", "uint8", "int64", "bf16", "fp16"]
    dname = names[rng.integers(len(names))]
    dtype = DTYPES[dname]
    es, npdt = N.DTYPE_SIZE[dtype], N.NP_DTYPE[dtype]
    n = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12]))
    count = int(rng.integers(0, 300000)) if rng.random() < 0.9 else int(rng.integers(0, 20))
    op = int(rng.choice([N.OP_SUM, N.OP_PROD, N.OP_MAX, N.OP_MIN]))
    order, algo = int(rng.integers(4)), int(rng.integers(2))
    nsl, nred = int(rng.choice([1, 2, 8])), int(rng.choice([0, 1, 3]))
    inplace = bool(rng.integers(2))
    kind = int(rng.integers(3))       # 0 all-reduce, 1 reduce, 2 reduce-scatter
    sixteen = dname in ("bf16", "fp16")
    if sixteen:                       # the chain oracles round at every step for 16-bit types: only rank order compares
        order, algo = S.ORDER_RANK, S.ALGO_DIRECT
    seed = int(rng.integers(1 << 30))
    desc = (f"case {no}: {dname} ranks={n} count={count} op={op} order={order} algo={algo} nslices={nsl} "
            f"nredslices={nred} inplace={inplace} kind={kind} seed={seed}")
    print(desc, flush=True)
    rank_order = order in (S.ORDER_RANK, S.ORDER_TREE) and algo == S.ALGO_DIRECT
    rc = count // n
    total = rc * n if kind == 2 else count
    sends = [a[:total] for a in seeded_inputs(dtype, n, max(total, 1), seed=seed)]
    with DevBufs(dev) as b, S.SimGroup(n, order=order, algo=algo, nslices=nsl, nredslices=nred, redslicesize=1024) as g:
        ds = [b.put(a, pad_after=64) for a in sends]
        if kind == 0:
            dr = ds if inplace else [b.alloc(count * es + 64) for _ in range(n)]
            N.check(g.all_reduce(ds, dr, count, dtype, op, stream), desc)
            dev.stream_sync(stream)
            if count == 0:
                return
            if rank_order:
                want = O.reduce_copy(sends, dtype, op)
            elif order == S.ORDER_HOST:
                want = O.bootstrap_allreduce(sends, dtype, op)[0] if n > 1 else sends[0]
            elif order == S.ORDER_RING or algo == S.ALGO_RING:
                want = O.ring_allreduce(sends, dtype, op)[0]
            else:
                want = O.reduce_copy(sends, dtype, op)
            for r in range(n):
                assert_parity(dev.to_host(dr[r], count, npdt), want, dtype, op, desc + f" rank {r}")
        elif kind == 1:
            root = int(rng.integers(n))
            dout = ds[root] if inplace else b.alloc(count * es + 64)
            N.check(g.reduce(ds, [dout if r == root else None for r in range(n)], count, dtype, op, root, stream), desc)
            dev.stream_sync(stream)
            if count == 0:
                return
            if order == S.ORDER_TREE and n > 1:
                want = O.tree_reduce(sends, root, dtype, op)
            elif order == S.ORDER_HOST and n > 1:
                want = O.bootstrap_allreduce(sends, dtype, op)[0]
            else:
                want = O.reduce_copy(sends, dtype, op)
            assert_parity(dev.to_host(dout, count, npdt), want, dtype, op, desc)
        else:
            if rc == 0:
                return
            dr = [b.alloc(rc * es + 64) for _ in range(n)]
            N.check(g.reduce_scatter(ds, dr, rc, dtype, op, stream), desc)
            dev.stream_sync(stream)
            for r in range(n):
                part = [a[r * rc:(r + 1) * rc] for a in sends]
                if n == 1:
                    want = part[0]
                elif rank_order:
                    want = O.reduce_copy(part, dtype, op)
                elif order == S.ORDER_HOST:
                    chain = ([part[(r - j) % n] for j in range(n)] if op in (N.OP_MAX, N.OP_MIN)
                             else [part[(r + 1 + j) % n] for j in range(n)])
                    want = O.reduce_copy(chain, dtype, op)
                elif order == S.ORDER_RING or algo == S.ALGO_RING:
                    want = O.reduce_copy(part, dtype, op, first=(r + 1) % n)
                else:
                    want = O.reduce_copy(part, dtype, op)
                assert_parity(dev.to_host(dr[r], rc, npdt), want, dtype, op, desc + f" rank {r}")


def test_collectives_random_cases(dev):
    rng = np.random.default_rng(20240612)
    stream = dev.stream_create()
    try:
        for no in range(1500):
            _collective_case(dev, stream, rng, no)
    finally:
        dev.stream_destroy(stream)


def _fifo_round(dev, rng, no):
    """One consumer launch on a ring of random capacity, one to three batches of
    random two-input triggers through the producer loop, then terminate."""
    lib = N.lib
    names = list(DTYPES)
    cap = int(rng.choice([1, 2, 3, 5, 16, 64, 128]))
    host = dev.malloc(lib.fx_fifo_bytes(cap), N.MEM_HOST)
    N.check(lib.fx_fifo_init(host, cap))
    dptr = C.c_void_p()
    N.check(dev.t.hostGetDevicePointer(C.byref(dptr), host))
    stream = dev.stream_create()
    cons = C.c_void_p()
    N.check(lib.fx_fifo_consumer_create(C.byref(cons), cap))
    # the idle limit (in polls of the host ring, each over a microsecond) has to outlast the host's own work
    # between batches -- uploads and the oracle; `terminate` is what ends the kernel
    N.check(lib.fx_fifo_consumer_launch(cons, dptr, host, 30_000_000, dev.raw_stream(stream)))
    total_done = 0
    with DevBufs(dev) as b:
        try:
            for batch_no in range(int(rng.integers(1, 4))):
                total = int(rng.integers(1, 100))
                trig = (N.ReduceTrigger * total)()
                cases = []
                for i in range(total):
                    dname = names[rng.integers(len(names))]
                    dtype = DTYPES[dname]
                    es = N.DTYPE_SIZE[dtype]
                    op = int(rng.integers(0, 5))
                    n = int(rng.choice([0, 1, 3, 100, 4097, 65536, 200003, 1500000]))
                    mis = [int(rng.integers(0, 4)) * es for _ in range(3)] if rng.random() < 0.3 else [0, 0, 0]
                    a, c = seeded_inputs(dtype, 2, max(n, 1), seed=int(rng.integers(1 << 30)))
                    da = b.alloc(max(n, 1) * es + 64) + mis[0]
                    dc = b.alloc(max(n, 1) * es + 64) + mis[1]
                    dev.upload(da, a)
                    dev.upload(dc, c)
                    do = da if rng.random() < 0.2 else b.alloc(max(n, 1) * es + 64) + mis[2]
                    lib.fx_trigger_set(C.byref(trig[i]), da, dc, do, n, 32, dtype, op, 1)
                    cases.append((dname, dtype, op, n, a, c, do))
                print(f"round {no}: capacity {cap}, batch {batch_no}, {total} triggers", flush=True)
                N.check(lib.fx_fifo_run_batch(host, trig, total, 300_000_000))
                total_done += total
                for i, (dname, dtype, op, n, a, c, do) in enumerate(cases):
                    if n:
                        assert_parity(dev.to_host(do, n, N.NP_DTYPE[dtype]), O.reduce2(a[:n], c[:n], dtype, op), dtype, op,
                                      f"round {no} batch {batch_no} trigger {i}: {dname} op={op} n={n}")
        finally:                          # before the buffers go: freeing device memory waits for running kernels
            lib.fx_fifo_terminate(host)
            dev.stream_sync(stream)
    reason, done, bad = C.c_int(-1), C.c_uint64(), C.c_uint64()
    N.check(lib.fx_fifo_consumer_status(cons, C.byref(reason), C.byref(done), C.byref(bad)))
    assert (reason.value, done.value, bad.value) == (1, total_done, 0)     # 1 = FX_FIFO_EXIT_TERMINATE
    lib.fx_fifo_consumer_destroy(cons)
    dev.stream_destroy(stream)
    dev.free(host, N.MEM_HOST)


def test_reduce_fifo_random_rounds(dev):
    rng = np.random.default_rng(20240613)
    for no in range(30):
        _fifo_round(dev, rng, no)
