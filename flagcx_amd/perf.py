"""Size / op sweeps in the style of FlagCX's perf harness
(test/perf_common.cc:140-239: warmup 5, iters 20, sizes min..max x factor,
algBw = bytes / 1e9 / t).  Usage:

    python -m flagcx_amd.perf reduce  -k 4 -d fp16 -o sum -b 1K -e 1G -f 2 [--inplace]
    python -m flagcx_amd.perf slices            # BASELINE.json configs[1]: rank shares in 512 KiB pieces + all-gather copy
    python -m flagcx_amd.perf pack              # BASELINE.json configs[3]: alltoallv pack / unpack
    python -m flagcx_amd.perf allreduce -n 8 -d bf16 -b 1M -e 64M [--graph]
    python -m flagcx_amd.perf fifo -b 4K -e 256M -f 8   # round trips through the reduce FIFO
    python -m flagcx_amd.perf coldstart         # library sizes and the first call's latency (code-object load)

Warm and cold.  Every figure is "warm" unless --cold is given: the same buffers
are used launch after launch, so whatever of them fits MI355X's 256 MiB
memory-side cache is served from it.  With --cold (reduce, slices, pack) every
timed launch is preceded by a 1 GiB fill with ordinary stores that pushes the
operands out of that cache, and is timed by its own pair of events; both
columns are printed.  reduce --fresh adds the case a reduction meets when it
follows the kernel that made its operands: the inputs rewritten just before
the timed launch, with the caches otherwise warm and after the 1 GiB fill.
"""
import argparse
import sys

import numpy as np

from . import _native as N
from . import kernels as K
from . import sim as S
from .adaptor import Device

DT = {"fp32": N.DT_FP32, "fp16": N.DT_FP16, "bf16": N.DT_BF16, "int32": N.DT_INT32, "uint32": N.DT_UINT32,
      "int8": N.DT_INT8, "uint8": N.DT_UINT8, "int64": N.DT_INT64, "uint64": N.DT_UINT64, "fp64": N.DT_FP64}
OP = {"sum": N.OP_SUM, "prod": N.OP_PROD, "max": N.OP_MAX, "min": N.OP_MIN, "avg": N.OP_AVG}


def size(s):
    mult = {"K": 1 << 10, "M": 1 << 20, "G": 1 << 30}
    return int(s[:-1]) * mult[s[-1].upper()] if s[-1].upper() in mult else int(s)


class Timer:
    def __init__(self, dev, warmup=5, iters=20):
        self.dev, self.warmup, self.iters = dev, warmup, iters
        self.stream = dev.stream_create()
        self.raw = dev.raw_stream(self.stream)

    def ms(self, fn):
        """Milliseconds per call: `iters` back-to-back calls between two events, the
        median of three such rounds (one host hiccup of half a millisecond would
        otherwise add tens of microseconds to a ten-microsecond figure)."""
        d = self.dev
        for _ in range(self.warmup):
            fn()
        d.stream_sync(self.stream)
        rounds = []
        for _ in range(3):
            e0, e1 = d.event_create(), d.event_create()
            d.event_record(e0, self.stream)
            for _ in range(self.iters):
                fn()
            d.event_record(e1, self.stream)
            d.event_sync(e1)
            rounds.append(d.event_ms(e0, e1) / self.iters)
            d.event_destroy(e0)
            d.event_destroy(e1)
        return sorted(rounds)[1]

    SCRUB_BYTES = 1 << 30

    def ms_cold(self, fn, launches=9, scrub=True, produce=None):
        """Milliseconds per call when the caches hold nothing of the operands: before
        every timed call a 1 GiB fill with ordinary stores (the runtime's memset
        kernel, four times the memory-side cache) runs on the same stream; each call
        is timed by its own pair of events; the median of `launches` calls.
        `produce` (a function that rewrites the inputs on the stream) runs after the
        fill and before the timed call: the inputs are then what a kernel has just
        written, as when a reduction follows the kernel that made its operands;
        `scrub=False` leaves the fill out."""
        d = self.dev
        if scrub and not hasattr(self, "scrub"):
            self.scrub = d.malloc(self.SCRUB_BYTES)
        fn()
        d.stream_sync(self.stream)
        each = []
        for i in range(launches):
            if scrub:
                d.memset(self.scrub, i & 0xff, self.SCRUB_BYTES, self.stream)
            if produce:
                produce()
            e0, e1 = d.event_create(), d.event_create()
            d.event_record(e0, self.stream)
            fn()
            d.event_record(e1, self.stream)
            d.event_sync(e1)
            each.append(d.event_ms(e0, e1))
            d.event_destroy(e0)
            d.event_destroy(e1)
        return sorted(each)[len(each) // 2]

    def both(self, fn, cold, produce=None):
        """(warm ms, cold ms or None), and with `produce` two more: (.., inputs just
        written, 1 GiB fill and then the inputs written)."""
        res = (self.ms(fn), (self.ms_cold(fn) if cold else None))
        if produce:
            res += (self.ms_cold(fn, scrub=False, produce=produce), self.ms_cold(fn, produce=produce))
        return res


def row(label, nbytes, ms, algo_bytes):
    """ms: milliseconds, or the tuple from Timer.both."""
    warm, cold = ms[:2] if isinstance(ms, tuple) else (ms, None)
    line = f"{label:<44s} size {nbytes:>12d} B   {warm * 1e3:10.2f} us   {algo_bytes / warm / 1e6:9.1f} GB/s"
    if cold is not None:
        line += f"   | cold {cold * 1e3:10.2f} us   {algo_bytes / cold / 1e6:9.1f} GB/s"
    if isinstance(ms, tuple) and len(ms) == 4:
        line += f"   | inputs fresh {ms[2] * 1e3:8.2f} us   | fill, then inputs fresh {ms[3] * 1e3:8.2f} us"
    print(line, flush=True)


def run_reduce(dev, a):
    t = Timer(dev)
    dtype, op, k = DT[a.dtype], OP[a.op], a.k
    es = N.DTYPE_SIZE[dtype]
    emax = size(a.max)
    if a.stride:        # one arena: buffer i starts i * stride bytes in (the output is buffer k), plus the shifts
        span = size(a.stride)
        arena = dev.malloc((k + 1) * span + emax + a.misalign * es + a.in_shift * k)
        ins = [arena + i * span + a.in_shift * i for i in range(k)]
        spare = arena + k * span
    else:
        ins = [dev.malloc(emax + a.misalign * es + a.in_shift * k) + a.in_shift * i for i in range(k)]
        spare = None
    for i, p in enumerate(ins):
        if a.fill == "uniform":      # seeded uniform(-1, 1) (integers: 0..99), another stream per input
            flt = dtype in (N.DT_FP16, N.DT_FP32, N.DT_FP64, N.DT_BF16)
            dev.upload(p, K.synth(emax // es, dtype, K.SYNTH_UNIFORM if flt else K.SYNTH_UNIFORM_INT,
                                  -1.0 if flt else 0.0, 1.0 if flt else 100.0, 7, i))
        else:
            dev.memset(p, 0 if a.fill == "zeros" else 0x3c + i, emax)
    out = ins[0] if a.inplace else (spare if spare is not None else dev.malloc(emax + a.misalign * es))
    nbytes = size(a.min)
    while nbytes <= emax:
        n = nbytes // es
        shift = [(a.misalign * es if a.mixed and i % 2 else 0) for i in range(k)]
        fn = lambda: N.check(K.reduce_copy(out + (0 if a.inplace else a.misalign * es),
                                           [p + (a.misalign * es if not a.mixed else s) for p, s in zip(ins, shift)]
                                           if not a.inplace else ins, n, dtype, op, 0, t.raw))
        produce = None
        if a.fresh and not a.inplace:      # the inputs rewritten by a fill of their own before every timed launch
            produce = lambda: [dev.memset(p, 0x3c + i, nbytes + a.misalign * es, t.stream) for i, p in enumerate(ins)]
        row(f"reduce k={k} {a.dtype} {a.op}{' inplace' if a.inplace else ''}", nbytes, t.both(fn, a.cold, produce),
            (k + 1) * nbytes)
        nbytes *= a.factor


def run_slices(dev, a):
    """Config 2: 8 peers x 33,554,432 bf16; each rank share (4,194,304 el) in 8 slices x 2 pieces of 512 KiB."""
    t = Timer(dev)
    k, n, es = 8, 33_554_432, 2
    ds = [dev.malloc(n * es) for _ in range(k)]
    dr = [dev.malloc(n * es) for _ in range(k)]
    for i, p in enumerate(ds):
        dev.memset(p, 0x3c + i, n * es)
    per_rank, copies = [], []
    for ch in range(k):
        ccnt, coff = K.split(n, k, ch)
        owner = (ch - 1) % k
        descs = []
        for s in range(8):
            scnt, soff = K.split(ccnt, 8, s)
            for q in range(2):
                rcnt, roff = K.split(scnt, 2, q)
                off = (coff + soff + roff) * es
                descs.append(([p + off for p in ds], dr[owner] + off, rcnt))
        per_rank.append(descs)
        copies += [(dr[owner] + coff * es, dr[r] + coff * es, ccnt * es) for r in range(k) if r != owner]
    share_bytes = n // k * es
    one = per_rank[0]
    # descriptor arrays are marshalled once, outside the timed calls: building 128 ctypes descriptors in Python
    # takes longer than the launch they describe
    def reducer(descs, kk=k):
        arr, cnt = K.make_slices(descs)
        return lambda: N.check(N.lib.fx_reduce_slices(arr, cnt, kk, N.DT_BF16, N.OP_SUM, t.raw))

    def copier(descs):
        arr, cnt = K.make_slices(([s], d, b) for s, d, b in descs)
        return lambda: N.check(N.lib.fx_copy_slices(arr, cnt, t.raw))

    row("one rank share: 16 x 512 KiB, 8-way", share_bytes, t.both(reducer(one), a.cold), 9 * share_bytes)
    allr = [d for r in per_rank for d in r]
    row("all 8 shares: 128 x 512 KiB, 8-way", n * es, t.both(reducer(allr), a.cold), 9 * n * es)
    plan = K.Plan(allr, k, N.DT_BF16, N.OP_SUM)
    row("all 8 shares as a device-resident plan", n * es, t.both(lambda: N.check(plan.launch(t.raw)), a.cold), 9 * n * es)
    onechunk = [([p for p in ds], dr[0], n // k)]
    row("one share as ONE contiguous slice", share_bytes, t.both(reducer(onechunk), a.cold), 9 * share_bytes)
    # ring-faithful: 7 successive 2-input steps over the share (reported, not the target)
    steps = [[([ds[0] + o, ds[1] + o], dr[0] + o, c) for (ins_, _, c), o in
              zip(one, [d[1] - dr[-1 % k] for d in one])]]
    two = [([d[0][0], d[0][1]], d[1], d[2]) for d in one]
    step = reducer(two, 2)
    row("ring-faithful: 7 x (16 x 512 KiB, 2-input)", share_bytes, t.ms(lambda: [step() for _ in range(7)]), 7 * 3 * share_bytes)
    one_rank_ag = [c for c in copies if c[1] - dr[0] >= 0 and c[1] - dr[0] < n * es]
    row("all-gather copy, one rank: 7 x 8 MiB", 7 * share_bytes, t.both(copier(one_rank_ag), a.cold), 2 * 7 * share_bytes)
    row("all-gather copy, all ranks: 56 x 8 MiB", 56 * share_bytes, t.both(copier(copies), a.cold), 2 * 56 * share_bytes)
    with S.SimGroup(k, nslices=8, redslicesize=262144) as g:
        row("flagcxAllReduce, 8 simulated ranks, 64 MiB", n * es,
            t.ms(lambda: N.check(g.all_reduce(ds, dr, n, N.DT_BF16, N.OP_SUM, t.stream))), 9 * n * es + 2 * 56 * share_bytes)


def run_pack(dev, a):
    from tests.golden import workloads as W
    t = Timer(dev)
    counts, sd, slen, rd, rlen = W.cfg4_layout()
    total = sum(counts)
    dsend, dpacked, drecv = dev.malloc(slen * 4), dev.malloc(total * 4), dev.malloc(rlen * 4)
    dev.memset(dsend, 1, slen * 4)
    print("counts", counts, "sdispls % 4 el:", [d % 4 for d in sd], "slots % 4:", [int(x) % 4 for x in np.cumsum([0] + counts[:-1])])
    row("pack   (config 4 layout)", total * 4, t.both(lambda: N.check(K.pack(dpacked, dsend, counts, sd, N.DT_FP32, t.raw)), a.cold), 2 * total * 4)
    row("unpack (config 4 layout)", total * 4, t.both(lambda: N.check(K.unpack(drecv, dpacked, counts, rd, N.DT_FP32, t.raw)), a.cold), 2 * total * 4)
    # the two phases as one step: two dependent launches, eagerly and as one replayed graph of two kernel nodes
    both = lambda: (N.check(K.pack(dpacked, dsend, counts, sd, N.DT_FP32, t.raw)),
                    N.check(K.unpack(drecv, dpacked, counts, rd, N.DT_FP32, t.raw)))
    row("pack + unpack, two launches", 2 * total * 4, t.ms(both), 4 * total * 4)
    row("pack + unpack, one graph of two nodes", 2 * total * 4, t.ms(_replay_of(t, both)), 4 * total * 4)
    row("4 x (pack + unpack), one graph", 8 * total * 4, t.ms(_replay_of(t, both, 4)), 16 * total * 4)
    c4 = [c // 4 * 4 for c in counts]
    s4 = [d // 4 * 4 for d in sd]
    row("pack, counts/displs multiples of 16 B", sum(c4) * 4, t.ms(lambda: N.check(K.pack(dpacked, dsend, c4, s4, N.DT_FP32, t.raw))), 2 * sum(c4) * 4)
    big = [4_194_304] * 8
    bd = [i * 4_194_304 + 0 for i in range(8)]
    dbig, dpk = dev.malloc(8 * 4_194_304 * 4 + 64), dev.malloc(8 * 4_194_304 * 4)
    dev.memset(dbig, 2, 8 * 4_194_304 * 4 + 64)
    row("pack, 8 x 4,194,304 el aligned", sum(big) * 4, t.both(lambda: N.check(K.pack(dpk, dbig, big, bd, N.DT_FP32, t.raw)), a.cold), 2 * sum(big) * 4)
    row("pack, 8 x 4,194,304 el, source off by 1 el", sum(big) * 4,
        t.ms(lambda: N.check(K.pack(dpk, dbig + 4, big, bd, N.DT_FP32, t.raw))), 2 * sum(big) * 4)


def run_fifo(dev, a):
    """Round trip through the reference's reduce FIFO with the persistent consumer:
    host enqueue -> kernel executes -> host sees Complete.  Wall-clock on the host."""
    import ctypes as C
    import time
    lib = N.lib
    cap = 128
    host = dev.malloc(lib.fx_fifo_bytes(cap), N.MEM_HOST)
    N.check(lib.fx_fifo_init(host, cap))
    dptr = C.c_void_p()
    N.check(dev.t.hostGetDevicePointer(C.byref(dptr), host))
    stream = dev.stream_create()
    cons = C.c_void_p()
    N.check(lib.fx_fifo_consumer_create(C.byref(cons), cap))
    N.check(lib.fx_fifo_consumer_launch(cons, dptr, host, 20_000_000, dev.raw_stream(stream)))
    emax = size(a.max)
    bufs = [dev.malloc(emax) for _ in range(3)]
    for i, p in enumerate(bufs):
        dev.memset(p, 0x3c + i, emax)
    idx = C.c_int()

    def one(n):
        while True:
            lib.fx_fifo_enqueue(host, bufs[0], bufs[1], bufs[2], n, 32, N.DT_FP32, N.OP_SUM, C.byref(idx))
            if idx.value >= 0:
                break
        while lib.fx_fifo_poll_state(host, idx.value) != 3:
            pass
        lib.fx_fifo_set_state(host, idx.value, 0)

    try:
        nbytes = size(a.min)
        while nbytes <= emax:
            n = nbytes // 4
            for _ in range(5):
                one(n)
            t0 = time.perf_counter()
            for _ in range(20):
                one(n)
            ms = (time.perf_counter() - t0) * 1e3 / 20
            row("fifo round trip, fp32 sum, 2 inputs", nbytes, ms, 3 * nbytes)
            # the ring kept full: 1024 independent triggers through the library's own producer loop
            # (enqueue as slots free up, collect as they complete)
            windows = min(64, emax // nbytes)                    # disjoint windows of the buffers
            if windows >= 2:
                span = emax // (windows * 4) * 4
                n = min(n, span // 4)
                total = max(32, min(1024, (8 << 30) // (3 * nbytes)))
                trig = (N.ReduceTrigger * total)()
                for i in range(total):
                    off = (i % windows) * span
                    lib.fx_trigger_set(C.byref(trig[i]), bufs[0] + off, bufs[1] + off, bufs[2] + off, n, 32, N.DT_FP32,
                                       N.OP_SUM, 1)
                N.check(lib.fx_fifo_run_batch(host, trig, min(64, total), 50_000_000))          # warm-up
                t0 = time.perf_counter()
                N.check(lib.fx_fifo_run_batch(host, trig, total, 50_000_000))
                ms = (time.perf_counter() - t0) * 1e3 / total
                row("fifo ring kept full, per trigger", n * 4, ms, 3 * n * 4)
            nbytes *= a.factor
        # BASELINE.json configs[1] as the reference's scheduler would run it through this ring: one reduce-scatter step of
        # the ring all-reduce for all 8 simulated ranks = 8 x 8 slices x 2 pieces = 128 two-input bf16 triggers of
        # 262,144 elements (512 KiB), all independent; 7 such steps make the reduce-scatter.
        n, k, piece = 33_554_432, 8, 262_144
        if emax >= n * 2:
            chunk = n // k
            total = k * (chunk // piece)
            trig = (N.ReduceTrigger * total)()
            t = 0
            for r in range(k):
                for q in range(chunk // piece):
                    off = (r * chunk + q * piece) * 2
                    lib.fx_trigger_set(C.byref(trig[t]), bufs[0] + off, bufs[1] + off, bufs[2] + off, piece, 32,
                                       N.DT_BF16, N.OP_SUM, 1)
                    t += 1
            N.check(lib.fx_fifo_run_batch(host, trig, total, 50_000_000))          # warm-up
            t0 = time.perf_counter()
            for _ in range(7):
                N.check(lib.fx_fifo_run_batch(host, trig, total, 50_000_000))
            ms = (time.perf_counter() - t0) * 1e3 / 7
            row("config-2 ring step, 128 triggers of 512 KiB", total * piece * 2, ms, 3 * total * piece * 2)
    finally:
        lib.fx_fifo_terminate(host)
        dev.stream_sync(stream)
        lib.fx_fifo_consumer_destroy(cons)


def _replay_of(t, post, calls=1):
    """Capture what `calls` calls of `post` enqueue on the timer's stream into a HIP graph once; the returned
    function replays it."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so.7")          # the runtime the library is linked against (same mapping)
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    graph, gexec = C.c_void_p(), C.c_void_p()
    post()                                    # first call outside the capture: one-time set-up
    t.dev.stream_sync(t.stream)
    if hip.hipStreamBeginCapture(t.raw, 0) != 0:
        raise RuntimeError("hipStreamBeginCapture failed")
    try:
        for _ in range(calls):
            post()
    finally:
        rc = hip.hipStreamEndCapture(t.raw, C.byref(graph))
    if rc != 0 or hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) != 0:
        raise RuntimeError("the call could not be captured into a graph")

    def replay():
        if hip.hipGraphLaunch(gexec, t.raw) != 0:
            raise RuntimeError("hipGraphLaunch failed")
    return replay                             # graph and executable live until the process ends


def run_allreduce(dev, a):
    t = Timer(dev)
    dtype, n = DT[a.dtype], a.nranks
    es = N.DTYPE_SIZE[dtype]
    emax = size(a.max)
    ds = [dev.malloc(emax) for _ in range(n)]
    dr = [dev.malloc(emax) for _ in range(n)]
    for algo in (S.ALGO_DIRECT, S.ALGO_RING):
        with S.SimGroup(n, algo=algo) as g:
            nbytes = size(a.min)
            while nbytes <= emax:
                cnt = nbytes // es
                post = lambda: N.check(g.all_reduce(ds, dr, cnt, dtype, OP[a.op], t.stream))
                ms = t.ms(_replay_of(t, post, a.graph_calls)) / a.graph_calls if a.graph else t.ms(post)
                alg = nbytes / ms / 1e6
                # algBw = size / time, busBw = algBw * 2 (n - 1) / n, as test/perf/host_api/test_allreduce.cpp:11
                print(f"{'allreduce n=%d %s %s' % (n, a.dtype, ('ring' if algo else 'direct') + (' graph' if a.graph else '')):<44s} size {nbytes:>12d} B   "
                      f"{ms * 1e3:10.2f} us   algBw {alg:9.1f} GB/s   busBw {alg * 2 * (n - 1) / n:9.1f} GB/s", flush=True)
                nbytes *= a.factor


def run_collectives(dev, a):
    """Every reducing / gathering collective over n simulated ranks, per order and algorithm, at one size per rank:
    time per collective and TB/s of the least traffic the collective can do on one GPU."""
    t = Timer(dev, warmup=2, iters=5)
    per_rank = size(a.min)
    dtype = DT[a.dtype]
    es = N.DTYPE_SIZE[dtype]
    orders = {S.ORDER_RANK: "rank", S.ORDER_RING: "ring", S.ORDER_TREE: "tree", S.ORDER_HOST: "host"}
    print(f"{a.dtype}, {per_rank} B per rank; TB/s of: all-reduce (k+n) x size, reduce (n+1) x size, reduce-scatter (n+1) x size, "
          f"all-gather (1+n) x size  [size = bytes per rank]")
    for n in (2, 4, 8, 12, 16):
        count = per_rank // es
        ds = [dev.malloc(per_rank) for _ in range(n)]
        dr = [dev.malloc(per_rank) for _ in range(n)]
        for p in ds:
            dev.memset(p, 1, per_rank)
        for algo in (S.ALGO_DIRECT, S.ALGO_RING):
            for order, oname in orders.items():
                with S.SimGroup(n, algo=algo, order=order) as g:
                    rc = count // n
                    ms = [t.ms(lambda: N.check(g.all_reduce(ds, dr, count, dtype, OP[a.op], t.stream))),
                          t.ms(lambda: N.check(g.reduce(ds, [dr[0]] + [None] * (n - 1), count, dtype, OP[a.op], 0, t.stream))),
                          t.ms(lambda: N.check(g.reduce_scatter(ds, dr, rc, dtype, OP[a.op], t.stream))),
                          t.ms(lambda: N.check(g.all_gather(ds, dr, rc, dtype, t.stream)))]
                units = [2 * n, n + 1, n + 1, 1 + n]
                cells = "  ".join(f"{m * 1e3:8.1f} us {u * per_rank / m / 1e9:5.2f}" for m, u in zip(ms, units))
                print(f"n={n:2d} {'ring  ' if algo else 'direct'} {oname:4s} | all-reduce, reduce, reduce-scatter, all-gather: {cells}",
                      flush=True)
        for p in ds + dr:
            dev.free(p)


def run_torchref():
    """PyTorch's own kernels on the same shapes, as a reference point on the same box: torch.add(out=) for the
    two-input sum, Tensor.copy_ for the copy, and the 8-input bf16 sum done the torch way.  Uses torch only."""
    import torch
    torch.cuda.set_device(0)

    def ms_of(fn, iters):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            e1.synchronize()
            best = min(best, e0.elapsed_time(e1) / iters)
        return best

    scrub = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")

    def cold_ms_of(fn, launches=9):
        """As Timer.ms_cold: every launch behind a 1 GiB fill, timed by its own pair of events; the median."""
        each = []
        for i in range(launches):
            scrub.fill_(i)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            e1.synchronize()
            each.append(e0.elapsed_time(e1))
        return sorted(each)[len(each) // 2]

    for dt, es in ((torch.float32, 4), (torch.bfloat16, 2)):
        for mib in (16, 64, 256, 512):
            n = (mib << 20) // es
            a, b = torch.randn(n, device="cuda").to(dt), torch.randn(n, device="cuda").to(dt)
            c = torch.empty_like(a)
            add, copy = (lambda: torch.add(a, b, out=c)), (lambda: c.copy_(a))
            row(f"torch.add(a, b, out=c) {str(dt)[6:]}", mib << 20, (ms_of(add, 50), cold_ms_of(add)), 3 * (mib << 20))
            row(f"c.copy_(a) {str(dt)[6:]}", mib << 20, (ms_of(copy, 50), cold_ms_of(copy)), 2 * (mib << 20))
            del a, b, c
    n = (512 << 20) // 2
    xs = [torch.randn(n, device="cuda").to(torch.bfloat16) for _ in range(8)]
    out = torch.empty_like(xs[0])

    def chain():
        torch.add(xs[0], xs[1], out=out)
        for x in xs[2:]:
            out.add_(x)
    row("8 x bf16 as 7 torch adds (one-pass bytes)", 512 << 20, ms_of(chain, 10), 9 * (512 << 20))
    st = torch.stack(xs)
    row("torch.sum(stacked [8, n] bf16, 0, out=)", 512 << 20, ms_of(lambda: torch.sum(st, 0, out=out), 10), 9 * (512 << 20))


COLDSTART_CHILD = r"""
import ctypes as C, json, os, sys, time
t0 = time.perf_counter()
from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from flagcx_amd.adaptor import Device
t_import = time.perf_counter() - t0
dev = Device(0)
n = 1 << 20
out = {"import_and_dlopen_ms": round(t_import * 1e3, 2), "first_calls": []}
t0 = time.perf_counter()
bufs = [dev.malloc(n * 8) for _ in range(3)]
dev.sync()
out["runtime_init_and_3_mallocs_ms"] = round((time.perf_counter() - t0) * 1e3, 2)
for name, dt in (("bf16", N.DT_BF16), ("bf16 again", N.DT_BF16), ("fp32", N.DT_FP32), ("uint8", N.DT_UINT8), ("copy", None)):
    t0 = time.perf_counter()
    if dt is None:
        N.check(K.copy_slices([(bufs[0], bufs[2], n)]))
    else:
        N.check(K.reduce_copy(bufs[2], bufs[:2], n, dt, N.OP_SUM))
    dev.sync()
    out["first_calls"].append({"what": name, "ms": round((time.perf_counter() - t0) * 1e3, 3)})
print(json.dumps(out))
"""


def run_coldstart():
    """Sizes of the libraries and what the first call of a kind costs in a fresh
    process: every element type is a code object of its own inside
    libflagcx-kernels-mi355x.so, loaded (and decompressed) by the HIP runtime at the
    first launch of one of its kernels."""
    import json
    import os
    import subprocess
    for f in sorted(os.listdir(N.LIB_DIR)):
        print(f"{f:<36s} {os.path.getsize(os.path.join(N.LIB_DIR, f)) / (1 << 20):8.2f} MiB")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for run in range(3):
        r = subprocess.run([sys.executable, "-c", COLDSTART_CHILD], capture_output=True, text=True, cwd=root)
        if r.returncode != 0:
            print(r.stdout + r.stderr)
            return 1
        o = json.loads(r.stdout.strip().splitlines()[-1])
        calls = "  ".join(f"{c['what']} {c['ms']:.2f}" for c in o["first_calls"])
        print(f"fresh process {run}: import+dlopen {o['import_and_dlopen_ms']:.1f} ms, runtime init + 3 mallocs "
              f"{o['runtime_init_and_3_mallocs_ms']:.1f} ms, first calls (ms incl. sync): {calls}", flush=True)
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("what", choices=["reduce", "slices", "pack", "allreduce", "fifo", "collectives", "torchref", "coldstart"])
    ap.add_argument("--cold", action="store_true",
                    help="reduce / slices / pack: also time every launch after a 1 GiB fill that empties the caches")
    ap.add_argument("--fresh", action="store_true",
                    help="reduce: two more columns, every launch timed right after its inputs were rewritten on the "
                         "same stream -- without and with the 1 GiB fill before that")
    ap.add_argument("--fill", default="const", choices=["const", "zeros", "uniform"],
                    help="reduce: what the inputs hold -- byte 0x3c + i in input i (default), zeros, or seeded uniform values "
                         "(all-zero buffers run faster: 3 %% from memory, 12 %% from the caches)")
    ap.add_argument("-k", type=int, default=4)
    ap.add_argument("-n", "--nranks", type=int, default=8)
    ap.add_argument("-d", "--dtype", default="fp32", choices=list(DT))
    ap.add_argument("-o", "--op", default="sum", choices=list(OP))
    ap.add_argument("-b", "--min", default="1M")
    ap.add_argument("-e", "--max", default="1G")
    ap.add_argument("-f", "--factor", type=int, default=2)
    ap.add_argument("--inplace", action="store_true")
    ap.add_argument("--graph", action="store_true", help="allreduce: capture one call into a HIP graph and time replays")
    ap.add_argument("--graph-calls", type=int, default=1, help="allreduce --graph: calls captured into the one graph")
    ap.add_argument("--misalign", type=int, default=0, help="shift buffers by this many elements")
    ap.add_argument("--mixed", action="store_true", help="shift only every other input (inputs not aligned like the output)")
    ap.add_argument("--stride", default="",
                    help="reduce: place the k inputs and the output in ONE allocation, STRIDE bytes apart (e.g. 512M, 16G)")
    ap.add_argument("--in-shift", type=int, default=0,
                    help="start input i at byte offset i*IN_SHIFT of its allocation (multiple of 16 keeps vector loads)")
    a = ap.parse_args(argv)
    if a.what == "torchref":         # torch brings its own HIP runtime: nothing of this library is loaded beside it
        return run_torchref()
    if a.what == "coldstart":
        return run_coldstart()
    dev = Device(0)
    {"reduce": run_reduce, "slices": run_slices, "pack": run_pack, "allreduce": run_allreduce,
     "fifo": run_fifo, "collectives": run_collectives}[a.what](dev, a)


if __name__ == "__main__":
    sys.exit(main())
