#!/usr/bin/env python3
"""Benchmark of the k-way reduce-copy path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg5|cfg1|cfg2|cfg3|cfg4]

The default workload, cfg5, is the headline of BASELINE.json: achieved HBM GB/s of
the bf16 sum of 8 inputs x 512 MiB with fp32 accumulate.  One "step" is one pass
of the hot path over one batch: one fx_reduce_copy of 8 x 268,435,456 bf16
elements into a ninth buffer.  Inputs are resident in HBM before the timed
region.  Prints ONE JSON line; besides the headline it carries a compact
"configs" object with BASELINE.json's other four configurations (GB/s, fraction
of peak, parity against the committed oracle digests).

--workload cfgN measures configuration N alone with the same schema (value,
roofline, parity, cpu_baseline where the reference has a CPU path for it):
  cfg1  fp32 sum of two 64 MiB inputs -- the reference's own CPU-runnable case
  cfg2  8 peers x 33,554,432 bf16: all rank shares in 512 KiB pieces, 8-way, then the all-gather copy phase
  cfg3  4 inputs, 1 KiB .. 1 GiB, sum/max/min/prod on fp16/fp32/int32, out of place and in place
  cfg4  alltoallv pack / unpack of 8 peers' fp32 segments
"""
import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published peak
# HBM bytes per launch of the headline kernel come from two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE), each scaled by the same counter's reading for a
# plain copy of known size.  This run does not collect counters: the figure is
# read from the committed summary of those runs and the JSON line names it.
TRAFFIC_SOURCE = "profiles/reduceCopyDirect_bf16_sum_k8_512MiB.txt"
GOLDEN_JSON = os.path.join("tests", "golden", "golden.json")
GOLDEN_KEY = "cfg5_bf16_sum_8x268435456"
K_INPUTS = 8
ELEMS = 268_435_456            # per input: 512 MiB of bf16
SEED = 4                       # values N(0, 0.02)


def carried_traffic():
    """(bytes per launch, source) from the line 'traffic per launch = N B' of the
    profile summary, or (None, None) when the summary is not there."""
    import re
    try:
        text = open(os.path.join(ROOT, TRAFFIC_SOURCE)).read()
    except OSError:
        return None, None
    m = re.search(r"traffic per launch = ([0-9,]+) B", text)
    return (int(m.group(1).replace(",", "")), TRAFFIC_SOURCE) if m else (None, None)


def golden():
    try:
        return json.load(open(os.path.join(ROOT, GOLDEN_JSON)))
    except (OSError, ValueError):
        return {}


def golden_digest():
    return golden().get(GOLDEN_KEY, {}).get("out_sha256")


def sha(arr):
    import numpy as np
    return hashlib.sha256(np.ascontiguousarray(arr).view(np.uint8)).hexdigest()


def host_threads():
    return min(16, len(os.sched_getaffinity(0)))


class StreamTimer:
    """HIP events on the stream the launches go to."""

    def __init__(self, dev):
        self.dev = dev
        self.stream = dev.stream_create()
        self.raw = dev.raw_stream(self.stream)

    def ms(self, fn, steps, warmup):
        """(wall ms per step, event ms per step) of `steps` back-to-back calls."""
        d = self.dev
        for _ in range(warmup):
            fn()
        d.stream_sync(self.stream)
        e0, e1 = d.event_create(), d.event_create()
        t0 = time.perf_counter()
        d.event_record(e0, self.stream)
        for _ in range(steps):
            fn()
        d.event_record(e1, self.stream)
        d.stream_sync(self.stream)
        wall = (time.perf_counter() - t0) * 1e3 / steps
        ev = d.event_ms(e0, e1) / steps
        d.event_destroy(e0)
        d.event_destroy(e1)
        return wall, ev

    def close(self):
        self.dev.stream_destroy(self.stream)


def roofline(kernel, algo_bytes, kern_ms, **extra):
    gbs = algo_bytes / kern_ms / 1e6
    r = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
         "traffic": None, "kernel": kernel, "bytes_per_launch": algo_bytes, "avg_launch_ms": round(kern_ms, 4)}
    r.update(extra)
    return r


def line(metric, wall_ms, algo_bytes, steps, warmup, dtype, workload, roof, **extra):
    gbs = algo_bytes / wall_ms / 1e6
    r = {"metric": metric, "value": round(gbs, 1), "unit": "GB/s", "pct_of_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
         "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(wall_ms, 4), "higher_is_better": True,
         "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": workload, "roofline": roof}
    r.update(extra)
    return r


# --------------------------------------------------------------------- cfg1

def cfg1(args, dev=None):
    """BASELINE.json configs[0]: out = a + b, fp32, 16,777,216 elements, uniform[-1,1)
    seed 0 -- on the GPU and, as the reference runs it, as one scalar host loop.
    Returns the result object."""
    import numpy as np

    from flagcx_amd import _native as N
    from flagcx_amd import kernels as K
    from flagcx_amd.adaptor import Device

    n, k = 16_777_216, 2
    dev = dev or Device(0)
    threads = host_threads()
    host = [K.synth(n, N.DT_FP32, K.SYNTH_UNIFORM, -1.0, 1.0, 0, p, threads) for p in range(k)]
    dins = [dev.malloc(n * 4) for _ in range(k)]
    for d, h in zip(dins, host):
        dev.upload(d, h)
    out = dev.malloc(n * 4)
    t = StreamTimer(dev)
    algo_bytes = (k + 1) * n * 4
    wall_ms, kern_ms = t.ms(lambda: N.check(K.reduce_copy(out, dins, n, N.DT_FP32, N.OP_SUM, 0, t.raw), "fx_reduce_copy"),
                            args.steps, args.warmup)
    got = dev.to_host(out, n, np.float32)
    want_digest = golden().get("cfg1_fp32_sum_2x16777216", {}).get("out_sha256")
    result = line(
        "achieved HBM GB/s (% of peak) for 2-input reduce-copy, fp32 64 MiB", wall_ms, algo_bytes, args.steps, args.warmup, "f32",
        {"workload": "BASELINE configs[0]: fp32 sum, 2 inputs x 16,777,216 elements (64 MiB each), "
                     "uniform[-1,1) seed 0, out-of-place, one launch per step",
         "inputs": k, "elements_per_input": n, "op": "sum"},
        roofline("reduceCopyDirect<Red<fp32,sum>,2,2>", algo_bytes, kern_ms,
                 note="201 MB per launch fits the 256 MiB memory-side cache: repeated launches are cache assisted"),
        parity="bit-exact" if sha(got) == want_digest else "MISMATCH")
    if not args.no_cpu_baseline:
        from oracle import fx_oracle as O

        want = np.zeros(n, np.float32)           # touched before timing

        def best(nthreads, reps):
            O.lib.oracle_set_threads(nthreads)
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter()
                rc = O.lib.oracle_reduce2(want.ctypes.data, host[0].ctypes.data, host[1].ctypes.data, n, N.DT_FP32,
                                          N.OP_SUM)
                ts.append(time.perf_counter() - t0)
                assert rc == 0
            O.lib.oracle_set_threads(1)
            return min(ts), want

        t1, want = best(1, 5)
        tn, _ = best(threads, 5)
        if not np.array_equal(got.view(np.uint32), want.view(np.uint32)):
            result["parity"] = "MISMATCH"
        result["cpu_baseline"] = {
            "value": round(algo_bytes / t1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "the whole workload: one c[i] = a[i] + b[i] pass over the same two host arrays into a "
                      "resident third, best of 5",
            "all_cores": {"value": round(algo_bytes / tn / 1e9, 3), "cores": threads}}
        # The reference's CPU path END TO END for the same two buffers as two ranks' send buffers: what
        # FLAGCX_USE_HOST_COMM=1 costs per all-reduce (device to host, ring all-reduce with those loops, host to
        # device), with its own phase timers.  The library's C++ code, not the oracle.
        from flagcx_amd import sim as S
        outs = [out, dev.malloc(n * 4)]
        with S.HostStaged(k, dev.t.deviceMemcpy) as hs:
            hs.all_reduce(dins, outs, n, N.DT_FP32, N.OP_SUM)            # first call allocates the staged buffers
            t0 = time.perf_counter()
            rc, timers = hs.all_reduce(dins, outs, n, N.DT_FP32, N.OP_SUM)
            wall = time.perf_counter() - t0
        N.check(rc, "fxHostStagedAllReduce")
        staged = dev.to_host(outs[1], n, np.float32)
        dev.free(outs[1])
        result["cpu_baseline"]["host_staged_allreduce"] = {
            "what": "hostRunnerAllReduce shape (flagcx/runner/host_runner.cc:236-289): 2 simulated ranks, one host "
                    "thread each, sync D2H, bootstrap ring all-reduce on the host, sync H2D; second call (buffers warm)",
            "wall_ms": round(wall * 1e3, 3),
            "phases_ms_slowest_rank": {name: round(max(tm[name] for tm in timers) / 1e6, 3) for name in N.TIMER_NAMES},
            "parity": "bit-exact" if np.array_equal(staged.view(np.uint32), want.view(np.uint32)) else "MISMATCH",
            "gpu_us_same_arithmetic": round(kern_ms * 1e3, 2)}
    for p in dins + [out]:
        dev.free(p)
    t.close()
    return result


def reference_case(dev, threads):
    """The reference's own CPU-runnable case (BASELINE configs[0]) in short form,
    for the default line: its arithmetic on its own types -- the fp32
    c[i] = a[i] + b[i] loop of flagcx/service/include/utils.h:697-705 -- on one
    host core and on all of them, with the GPU launch beside it."""
    class A:
        steps, warmup, no_cpu_baseline = 50, 10, False
    r = cfg1(A, dev)
    return r, {"kind": "reference-semantics", "workload": r["config"]["workload"],
               "loop": "sum<float>, flagcx/service/include/utils.h:697-705 (restated in oracle/fx_oracle.c)",
               "cpu_GBs_1_core": r["cpu_baseline"]["value"], "cpu_GBs_all_cores": r["cpu_baseline"]["all_cores"]["value"],
               "cores": r["cpu_baseline"]["all_cores"]["cores"], "gpu_us_per_launch": round(r["roofline"]["avg_launch_ms"] * 1e3, 2),
               "gpu_GBs": r["roofline"]["achieved"], "bytes": r["roofline"]["bytes_per_launch"], "parity": r["parity"],
               "host_staged_allreduce": r["cpu_baseline"]["host_staged_allreduce"]}


# --------------------------------------------------------------------- cfg2

def cfg2(args, dev=None):
    """BASELINE.json configs[1]: 8 simulated peers x 33,554,432 bf16 N(0,1) seed 1.
    Step = every rank's reduce-scatter share (chunk of 4,194,304 elements in 8
    slices x 2 pieces of 512 KiB: 128 eight-input descriptors in ONE
    fx_reduce_slices call) followed by the all-gather copy phase (56 copies of
    8 MiB in ONE fx_copy_slices call).  value = the reduce phase; the copy phase
    and the sum of both are reported beside it."""
    import numpy as np

    from flagcx_amd import _native as N
    from flagcx_amd import kernels as K
    from flagcx_amd.adaptor import Device
    from tests.golden import workloads as W

    dev = dev or Device(0)
    c = W.CFG2
    n, k, es = c["n"], c["k"], 2
    threads = host_threads()
    ins = W.inputs(c["dtype"], k, n, c["dist"], c["seed"], threads)
    ds = [dev.to_device(a) for a in ins]
    dr = [dev.malloc(n * es) for _ in range(k)]
    nred = N.lib.fx_nredslices(n, k, c["nslices"], 0, c["redslice_elems"])
    descs, copies = [], []
    for ch in range(k):
        ccnt, coff = K.split(n, k, ch)
        owner = (ch - 1) % k
        for s in range(c["nslices"]):
            scnt, soff = K.split(ccnt, c["nslices"], s)
            for q in range(nred):
                rcnt, roff = K.split(scnt, nred, q)
                off = (coff + soff + roff) * es
                descs.append(([p + off for p in ds], dr[owner] + off, rcnt))
        copies += [([dr[owner] + coff * es], dr[r] + coff * es, ccnt * es) for r in range(k) if r != owner]
    t = StreamTimer(dev)
    rarr, rcnt_ = K.make_slices(descs)           # marshalled once: building 128 ctypes descriptors costs more than the launch
    carr, ccnt_ = K.make_slices(copies)
    reduce_fn = lambda: N.check(N.lib.fx_reduce_slices(rarr, rcnt_, k, c["dtype"], N.OP_SUM, t.raw), "fx_reduce_slices")
    copy_fn = lambda: N.check(N.lib.fx_copy_slices(carr, ccnt_, t.raw), "fx_copy_slices")
    red_bytes = (k + 1) * n * es                 # every share: 8 inputs read, one output written
    ag_bytes = 2 * len(copies) * (n // k) * es   # every copy: read + write
    ag_distinct = n * es + len(copies) * (n // k) * es   # each 8 MiB source once + every destination
    wall_r, kern_r = t.ms(reduce_fn, args.steps, args.warmup)
    wall_c, kern_c = t.ms(copy_fn, args.steps, args.warmup)
    wall_b, kern_b = t.ms(lambda: (reduce_fn(), copy_fn()), args.steps, args.warmup)
    gold = golden().get("cfg2_bf16_sum_8x33554432", {})
    digests = [sha(dev.to_host(dr[r], n, np.uint16)) for r in (0, 3, 7)]
    parity = "bit-exact" if gold.get("out_sha256") and all(d == gold["out_sha256"] for d in digests) else "MISMATCH"
    result = line(
        "achieved HBM GB/s (% of peak) for 8-way bf16 reduce-scatter shares in 512 KiB pieces, 8 peers x 64 MiB",
        wall_r, red_bytes, args.steps, args.warmup, "f32",
        {"workload": "BASELINE configs[1]: bf16 sum, 8 simulated peers x 33,554,432 elements, N(0,1) seed 1: all 8 rank shares "
                     "(8 slices x 2 pieces of 262,144 elements each: 128 descriptors, one call), then the all-gather copy phase "
                     "(56 copies of 8 MiB, one call)",
         "descriptors": len(descs), "red_slices_per_slice": int(nred), "copies": len(copies)},
        roofline("reduceSlicesInline<Red<bf16,sum>,8,4>", red_bytes, kern_r,
                 all_gather_copy={"kernel": "reduceSlicesInline<CopyRed<4>,1,2>", "bytes_per_launch": ag_distinct,
                                  "avg_launch_ms": round(kern_c, 4), "achieved": round(ag_distinct / kern_c / 1e6, 1),
                                  "frac": round(ag_distinct / kern_c / 1e6 / HBM_PEAK_GBS, 4),
                                  "copy_bytes": ag_bytes, "copy_GBs": round(ag_bytes / kern_c / 1e6, 1),
                                  "note": "each 8 MiB source is read by seven copies, six of them from a cache (ordinary loads "
                                          "for re-read sources): bytes_per_launch counts 64 MiB of distinct sources + 448 MiB "
                                          "written, copy_bytes the 2 x 56 x 8 MiB the copies move"},
                 both_phases={"avg_ms": round(kern_b, 4), "achieved": round((red_bytes + ag_bytes) / kern_b / 1e6, 1)}),
        parity=parity,
        parity_check="sha256 of ranks 0, 3 and 7's 64 MiB result after the timed launches == "
                     "tests/golden/golden.json[cfg2_bf16_sum_8x33554432].out_sha256")
    if not args.no_cpu_baseline:
        from oracle import fx_oracle as O
        ccnt, coff = K.split(n, k, 0)
        share = [a[coff:coff + ccnt] for a in ins]
        t0 = time.perf_counter()
        O.host_ring_passes(share, c["dtype"], N.OP_SUM)
        t1 = time.perf_counter() - t0
        result["cpu_baseline"] = {
            "value": round((k + 1) * ccnt * es / t1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"one rank share ({k} x {ccnt} bf16 elements), {k - 1} two-input passes on one core; the reference's host "
                      "path does not carry bf16 (flagcx/service/include/utils.h:690-694), so this is the oracle's loop"}
    for p in ds + dr:
        dev.free(p)
    t.close()
    return result


# --------------------------------------------------------------------- cfg3

def cfg3(args, dev=None, quick=False):
    """BASELINE.json configs[2]: 4 inputs, 1 KiB .. 1 GiB per input in powers of two,
    sum / max / min / prod on fp16 N(0,1), fp32 uniform[-1,1), int32
    uniform[-2^20, 2^20], out of place and in place (out = in[0]).  Every point up
    to 16 MiB is checked against the committed digest of the oracle's output, the
    largest against the oracle run live.  value = fp32 sum at the largest size.
    quick: three sizes (64 KiB, 16 MiB, 256 MiB), sum and max only."""
    import numpy as np

    from flagcx_amd import _native as N
    from flagcx_amd import kernels as K
    from flagcx_amd.adaptor import Device
    from tests.golden import workloads as W

    dev = dev or Device(0)
    k = W.CFG3["k"]
    threads = host_threads()
    gold = golden().get("cfg3", {})
    logs = [16, 24, 28] if quick else list(range(10, 31))
    ops = {"sum": N.OP_SUM, "max": N.OP_MAX} if quick else W.OPS
    max_bytes = 1 << logs[-1]
    t = StreamTimer(dev)
    points, checked, bad, live = {}, 0, [], 0
    head = None
    steps, warmup = (10, 3) if quick else (max(args.steps // 10, 5), max(args.warmup // 10, 2))
    for dtype in W.CFG3["dists"]:
        es = N.DTYPE_SIZE[dtype]
        name = W.DTYPE_NAMES[dtype]
        nmax = max_bytes // es
        ins = W.cfg3_inputs(dtype, nmax, threads)
        dins = [dev.to_device(a) for a in ins]
        dout, dwork = dev.malloc(nmax * es), dev.malloc(nmax * es)
        for oname, op in ops.items():
            oop, inp = [], []
            for lg in logs:
                n = (1 << lg) // es
                algo = (k + 1) * (1 << lg)
                _, ms_o = t.ms(lambda: N.check(K.reduce_copy(dout, dins, n, dtype, op, 0, t.raw)), steps, warmup)
                # in place: out = in[0]; runs on a copy of input 0 that is restored before the parity launch
                work = [dwork] + dins[1:]
                _, ms_i = t.ms(lambda: N.check(K.reduce_copy(dwork, work, n, dtype, op, 0, t.raw)), steps, warmup)
                oop.append(round(algo / ms_o / 1e6, 1))
                inp.append(round(algo / ms_i / 1e6, 1))
                want = gold.get(f"{name}_{oname}_{1 << lg}", {}).get("out_sha256")
                if want or lg == logs[-1]:
                    dev.copy(dwork, dins[0], n * es, t.stream)
                    N.check(K.reduce_copy(dwork, work, n, dtype, op, 0, t.raw))
                    dev.stream_sync(t.stream)
                    got_o, got_i = dev.to_host(dout, n, N.NP_DTYPE[dtype]), dev.to_host(dwork, n, N.NP_DTYPE[dtype])
                    if want:
                        checked += 2
                        bad += [f"{name} {oname} {1 << lg} {w}" for w, g in (("out-of-place", got_o), ("in-place", got_i))
                                if sha(g) != want]
                    elif not args.no_cpu_baseline:
                        from oracle import fx_oracle as O
                        O.lib.oracle_set_threads(threads)
                        ref = O.reduce_copy([a[:n] for a in ins], dtype, op)
                        O.lib.oracle_set_threads(1)
                        live += 2
                        bad += [f"{name} {oname} {1 << lg} {w} (live oracle)" for w, g in (("out-of-place", got_o), ("in-place", got_i))
                                if not np.array_equal(g.view(np.uint8), ref.view(np.uint8))]
                if dtype == N.DT_FP32 and oname == "sum" and lg == logs[-1]:
                    head = (algo, ms_o, n)
            points[f"{name}_{oname}"] = {"out_of_place_GBs": oop, "in_place_GBs": inp}
        for p in dins + [dout, dwork]:
            dev.free(p)
    algo, ms_o, n = head
    result = line(
        f"achieved HBM GB/s (% of peak) for 4-input reduce-copy, fp32 sum {max_bytes >> 20} MiB per input (size/op sweep)",
        ms_o, algo, steps, warmup, "f32",
        {"workload": "BASELINE configs[2]: 4 inputs, sizes 2^" + f"{logs[0]}..2^{logs[-1]} bytes per input, "
                     f"{'/'.join(ops)} on fp16 N(0,1), fp32 uniform[-1,1), int32 uniform[-2^20,2^20] (seed 2), out of place and in place",
         "log2_bytes_per_input": logs, "inputs": k},
        roofline("reduceCopyDirect<Red<fp32,sum>,4,4>", algo, ms_o),
        points=points,
        parity="bit-exact" if not bad and checked else "MISMATCH: " + "; ".join(bad[:5]),
        parity_check=f"{checked} outputs (every point up to 16 MiB per input, out of place and in place) == the committed "
                     f"oracle digests tests/golden/golden.json[cfg3]; {live} outputs at the largest size == the oracle run live")
    if not args.no_cpu_baseline and not quick:
        # the reference's host loops exist for fp32 / int32 sum, max, min (utils.h:664-725): k-1 two-input passes
        from oracle import fx_oracle as O
        ne = (64 << 20) // 4
        base = {}
        for dtype, dn in ((N.DT_FP32, "fp32"), (N.DT_INT32, "int32")):
            ins = W.cfg3_inputs(dtype, ne, threads)
            for oname in ("sum", "max", "min"):
                t0 = time.perf_counter()
                O.host_ring_passes(ins, dtype, W.OPS[oname])
                base[f"{dn}_{oname}"] = round((k + 1) * ne * 4 / (time.perf_counter() - t0) / 1e9, 3)
        result["cpu_baseline"] = {"value": base["fp32_sum"], "unit": "GB/s", "cores": 1, "kind": "port",
                                  "sample": "4 inputs x 64 MiB, 3 two-input passes of the host loop (utils.h:697-725) on one core, "
                                            "per type and op the reference's host path carries",
                                  "per_case_GBs": base}
    t.close()
    return result


# --------------------------------------------------------------------- cfg4

def cfg4(args, dev=None):
    """BASELINE.json configs[3]: alltoallv pack / unpack, 8 peers, fp32, per-peer
    counts log-uniform in [1, 4,194,304] from seed 3 with random displacements.
    Step = pack (gather the 8 segments into contiguous slots) + unpack (scatter
    them to the receive displacements); bytes = 2 x 2 x sum(counts) x 4."""
    import numpy as np

    from flagcx_amd import _native as N
    from flagcx_amd import kernels as K
    from flagcx_amd.adaptor import Device
    from tests.golden import workloads as W

    dev = dev or Device(0)
    threads = host_threads()
    e = golden().get("cfg4_alltoallv_pack_unpack", {})
    counts, sd, slen, rd, rlen = W.cfg4_layout()
    send = W.inputs(N.DT_FP32, 1, slen, (0, -1.0, 1.0), W.CFG4["seed"], threads)[0]
    total = sum(counts)
    dsend, dpacked, drecv = dev.to_device(send), dev.malloc(total * 4), dev.malloc(rlen * 4)
    dev.memset(drecv, 0, rlen * 4)
    t = StreamTimer(dev)
    pack = lambda: N.check(K.pack(dpacked, dsend, counts, sd, N.DT_FP32, t.raw), "fx_pack")
    unpack = lambda: N.check(K.unpack(drecv, dpacked, counts, rd, N.DT_FP32, t.raw), "fx_unpack")
    one = 2 * total * 4
    _, ms_p = t.ms(pack, args.steps, args.warmup)
    _, ms_u = t.ms(unpack, args.steps, args.warmup)
    wall, ms_b = t.ms(lambda: (pack(), unpack()), args.steps, args.warmup)
    packed, recv = dev.to_host(dpacked, total, np.float32), dev.to_host(drecv, rlen, np.float32)
    ok = sha(packed) == e.get("packed_sha256") and sha(recv) == e.get("unpacked_sha256")
    result = line(
        "achieved HBM GB/s (% of peak) for alltoallv pack + unpack, 8 peers fp32",
        wall, 2 * one, args.steps, args.warmup, "u32",
        {"workload": "BASELINE configs[3]: 8 peers, fp32, counts log-uniform in [1, 4,194,304] (seed 3), random displacements: "
                     "pack into contiguous slots, then unpack to the receive displacements",
         "counts": counts, "bytes_moved_per_phase": total * 4},
        roofline("reduceSlicesInline<CopyRed<4>,1,2>", 2 * one, ms_b,
                 pack={"avg_launch_ms": round(ms_p, 4), "achieved": round(one / ms_p / 1e6, 1)},
                 unpack={"avg_launch_ms": round(ms_u, 4), "achieved": round(one / ms_u / 1e6, 1)},
                 note="78 MB per phase fits the 256 MiB memory-side cache: repeated launches are cache assisted"),
        parity="bit-exact" if ok else "MISMATCH",
        parity_check="sha256 of the packed buffer and of the unpacked receive buffer == tests/golden/golden.json"
                     "[cfg4_alltoallv_pack_unpack]")
    if not args.no_cpu_baseline:
        # the reference moves each peer's segment with memcpy (self-copy of bootstrap.cc:1253-1258): the oracle's loop
        from oracle import fx_oracle as O
        t0 = time.perf_counter()
        p = O.pack(send, counts, sd)
        O.unpack(np.zeros(rlen, np.float32), p, counts, rd)
        t1 = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": round(2 * one / t1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                                  "sample": "the whole workload once: one memcpy per peer segment for pack and for unpack "
                                            "(flagcx/service/bootstrap.cc:1253-1258), one core"}
    for p_ in (dsend, dpacked, drecv):
        dev.free(p_)
    t.close()
    return result


def compact(r):
    """What the default line carries of another configuration."""
    o = {"GBs": r["roofline"]["achieved"], "frac": r["roofline"]["frac"], "us_per_launch": round(r["roofline"]["avg_launch_ms"] * 1e3, 2),
         "kernel": r["roofline"]["kernel"], "parity": r["parity"]}
    for extra in ("all_gather_copy", "pack", "unpack"):
        if extra in r["roofline"]:
            o[extra + "_GBs"] = r["roofline"][extra]["achieved"]
    return o


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--synthetic-fill", choices=["seeded", "memset"], default="seeded",
                    help="memset skips host generation (profiling runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a plain 512 MiB -> 512 MiB copy instead (known traffic, used to scale "
                         "the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--workload", choices=["cfg5", "cfg1", "cfg2", "cfg3", "cfg4"], default="cfg5",
                    help="cfg5 = the headline (default); cfg1..cfg4 = BASELINE.json's other configurations alone")
    ap.add_argument("--no-configs", action="store_true", help="cfg5: leave the compact cfg1..cfg4 object out (profiling runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus must be 1 "
              "(no collectives or second GPU are used anywhere in this run)", file=sys.stderr)
        sys.exit(2)

    if args.workload != "cfg5":
        r = {"cfg1": cfg1, "cfg2": cfg2, "cfg3": cfg3, "cfg4": cfg4}[args.workload](args)
        print(json.dumps(r))
        if "MISMATCH" in (r.get("parity", "")[:8], r.get("cpu_baseline", {}).get("host_staged_allreduce", {}).get("parity")):
            sys.exit(1)
        return

    from flagcx_amd import _native as N
    from flagcx_amd import kernels as K
    from flagcx_amd.adaptor import Device

    dev = Device(0)
    nbytes = ELEMS * 2
    if args.calibrate_copy:
        src, dst = dev.malloc(nbytes), dev.malloc(nbytes)
        dev.memset(src, 0x5a, nbytes)
        dev.sync()
        for _ in range(args.warmup + args.steps):
            N.check(K.copy_slices([(src, dst, nbytes)]), "fx_copy_slices")
        dev.sync()
        print(json.dumps({"calibration": "copy", "bytes_read_per_launch": nbytes, "bytes_written_per_launch": nbytes,
                          "launches": args.warmup + args.steps}))
        return
    threads = host_threads()
    ins, host_ins = [], []
    sample = ELEMS               # the CPU leg runs on the host copies of the whole inputs
    for p in range(K_INPUTS):
        d = dev.malloc(nbytes)
        if args.synthetic_fill == "seeded":
            host = K.synth(ELEMS, N.DT_BF16, K.SYNTH_NORMAL, 0.0, 0.02, SEED, p, threads)
            dev.upload(d, host)
            if not args.no_cpu_baseline:
                host_ins.append(host)
            del host
        else:
            dev.memset(d, 0x3c + p, nbytes)
        ins.append(d)
    out = dev.malloc(nbytes)
    t = StreamTimer(dev)
    stream, raw = t.stream, t.raw
    algo_bytes = (K_INPUTS + 1) * nbytes

    def step(dst):
        N.check(K.reduce_copy(dst, ins, ELEMS, N.DT_BF16, N.OP_SUM, 0, raw), "fx_reduce_copy")

    def per_launch(dst, steps):
        """Durations of individual launches: one event between consecutive steps."""
        ev = [dev.event_create() for _ in range(steps + 1)]
        dev.event_record(ev[0], stream)
        for i in range(steps):
            step(dst)
            dev.event_record(ev[i + 1], stream)
        dev.sync()
        ms = sorted(dev.event_ms(ev[i], ev[i + 1]) for i in range(steps))
        for e in ev:
            dev.event_destroy(e)
        return ms

    import numpy as np

    def digest_of(dptr):
        return sha(dev.to_host(dptr, ELEMS, np.uint16))

    wall_ms, kern_ms = t.ms(lambda: step(out), args.steps, args.warmup)
    each = per_launch(out, 20)
    # The buffer the timed launches wrote, against the committed digest of the CPU oracle's output for these inputs.
    want = golden_digest() if args.synthetic_fill == "seeded" else None
    parity = "not checked (no committed digest for this fill)"
    if want is not None:
        parity = "bit-exact" if digest_of(out) == want else "MISMATCH"
    _, inplace_ms = t.ms(lambda: step(ins[0]), max(args.steps // 2, 1), 2)      # out = in[0]; destroys input 0, run last
    traffic, traffic_source = carried_traffic()
    result = line(
        "achieved HBM GB/s (% of peak) for k-way reduce-copy, bf16 8-input 512 MiB", wall_ms, algo_bytes, args.steps, args.warmup,
        "f32",
        {"workload": "BASELINE configs[4]: bf16 sum reduce-copy, 8 inputs x 268,435,456 elements "
                     "(512 MiB each), N(0,0.02) seed 4, out-of-place, one launch per step",
         "inputs": K_INPUTS, "elements_per_input": ELEMS, "op": "sum", "storage": "bf16",
         "arithmetic": "every input widened to f32, f32 accumulate, one round-to-nearest-even to bf16",
         "in_place_GBs": round(algo_bytes / (inplace_ms * 1e-3) / 1e9, 1)},
        roofline("reduceCopyDirect<Red<bf16,sum>,8,4>", algo_bytes, kern_ms, traffic=traffic, traffic_source=traffic_source,
                 traffic_note="counter-measured in the profiling runs of that summary, not in this run",
                 min_launch_ms=round(each[0], 4), median_launch_ms=round(each[len(each) // 2], 4)),
        data="synthetic" if args.synthetic_fill == "seeded" else "synthetic (memset pattern)",
        parity=parity,
        parity_check="sha256 of the output buffer of the timed launches == tests/golden/golden.json"
                     f"[{GOLDEN_KEY}].out_sha256 (the CPU oracle's output for the same seeded inputs)")
    for p in ins + [out]:
        dev.free(p)
    t.close()
    mismatch = parity == "MISMATCH"
    if not args.no_cpu_baseline:
        if not host_ins:         # memset-filled profiling run: generate the sample now
            host_ins = [K.synth(sample, N.DT_BF16, K.SYNTH_NORMAL, 0.0, 0.02, SEED, p, threads) for p in range(K_INPUTS)]
        result["cpu_baseline"] = cpu_baseline(host_ins, threads)
    del host_ins
    if not args.no_configs and args.synthetic_fill == "seeded":
        # BASELINE.json's other configurations in short form (each alone, in full: --workload cfgN)
        class Short:
            steps, warmup, no_cpu_baseline = 50, 10, True
        r1, ref_case = reference_case(dev, threads) if not args.no_cpu_baseline else (cfg1(Short, dev), None)
        if ref_case:
            result["cpu_baseline"]["reference_case"] = ref_case
        short = {"cfg1": r1, "cfg2": cfg2(Short, dev), "cfg3": cfg3(Short, dev, quick=True), "cfg4": cfg4(Short, dev)}
        result["configs"] = {name: compact(r) for name, r in short.items()}
        result["configs"]["cfg3"]["note"] = "short form: 64 KiB, 16 MiB and 256 MiB per input, sum and max; the full sweep is --workload cfg3"
        result["configs"]["cfg3"]["points"] = short["cfg3"]["points"]
        mismatch = mismatch or any(r["parity"] != "bit-exact" for r in short.values())
    print(json.dumps(result))
    if mismatch:
        sys.exit(1)


def cpu_baseline(ins, threads_all):
    """The reference's host reduce path shape -- k-1 successive two-input passes
    over a running partial -- on the host copies of the same inputs, timed on
    this box's host cores (one pass on one core, ~7 s, two on all cores).  bf16 has no CPU
    path in the reference, so this is the oracle port."""
    from flagcx_amd import _native as N
    from oracle import fx_oracle as O

    k, sample_elems = len(ins), ins[0].size
    algo_bytes = (k + 1) * sample_elems * 2

    def best(threads, reps):
        O.lib.oracle_set_threads(threads)
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            O.host_ring_passes(ins, N.DT_BF16, N.OP_SUM)
            ts.append(time.perf_counter() - t0)
        O.lib.oracle_set_threads(1)
        return min(ts)

    t1 = best(1, 1)
    tn = best(threads_all, 2)
    return {
        "value": round(algo_bytes / t1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"{k} inputs x {sample_elems} bf16 elements (N(0,0.02), seed {SEED}), {k - 1} two-input passes, "
                  f"fp32 accumulate per pass, one run on one core; same (k+1)*size byte count as the GPU figure",
        "all_cores": {"value": round(algo_bytes / tn / 1e9, 3), "cores": threads_all},
    }


if __name__ == "__main__":
    main()
