"""FIFO-compatible consumer: the reference's reduce-trigger ring
(flagcx/core/flagcx_reduce_kernel_host.cc:46-98) driven exactly as its
scheduler drives it -- enqueue, poll for Complete, release the slot, terminate
-- with the persistent gfx950 kernel on the other end.  Every host wait has a
deadline and every kernel wait a poll limit, so nothing here can hang."""
import ctypes as C
import time

import numpy as np
import pytest

from flagcx_amd import _native as N
from oracle import fx_oracle as O
from tests.util import DevBufs, assert_parity, seeded_inputs

pytestmark = pytest.mark.gpu
lib = N.lib
AVAILABLE, ENQUEUED, INPROGRESS, COMPLETE = 0, 1, 2, 3
POLL_LIMIT = 4_000_000          # kernel-side bound: a few seconds of empty polls
DEADLINE = 20.0                 # host-side bound per wait, seconds


class Ring:
    """Pinned ring + consumer kernel on its own stream."""

    def __init__(self, dev, capacity, poll_limit=POLL_LIMIT):
        self.dev, self.cap = dev, capacity
        self.nbytes = lib.fx_fifo_bytes(capacity)
        self.host = dev.malloc(self.nbytes, N.MEM_HOST)
        N.check(lib.fx_fifo_init(self.host, capacity))
        dptr = C.c_void_p()
        N.check(dev.t.hostGetDevicePointer(C.byref(dptr), self.host))
        self.stream = dev.stream_create()
        self.consumer = C.c_void_p()
        N.check(lib.fx_fifo_consumer_create(C.byref(self.consumer), capacity))
        N.check(lib.fx_fifo_consumer_launch(self.consumer, dptr, self.host, poll_limit, dev.raw_stream(self.stream)))

    def words(self):
        return np.ctypeslib.as_array(C.cast(self.host, C.POINTER(C.c_uint64)), shape=(4,))

    def enqueue(self, in1, in2, out, count, dtype, op):
        idx = C.c_int(-1)
        t0 = time.time()
        while True:
            N.check(lib.fx_fifo_enqueue(self.host, in1, in2, out, count, 32, dtype, op, C.byref(idx)))
            if idx.value >= 0:
                return idx.value
            assert time.time() - t0 < DEADLINE, "ring never drained"

    def wait(self, idx):
        t0 = time.time()
        while lib.fx_fifo_poll_state(self.host, idx) != COMPLETE:
            assert time.time() - t0 < DEADLINE, f"trigger in slot {idx} never completed"
        N.check(lib.fx_fifo_set_state(self.host, idx, AVAILABLE))

    def close(self):
        """terminate -> the kernel drains and exits; returns (exitReason, completed, bad)."""
        lib.fx_fifo_terminate(self.host)
        self.dev.stream_sync(self.stream)
        reason, done, bad = C.c_int(-1), C.c_uint64(), C.c_uint64()
        N.check(lib.fx_fifo_consumer_status(self.consumer, C.byref(reason), C.byref(done), C.byref(bad)))
        lib.fx_fifo_consumer_destroy(self.consumer)
        self.dev.stream_destroy(self.stream)
        self.dev.free(self.host, N.MEM_HOST)
        return reason.value, done.value, bad.value


def test_triggers_through_the_ring(dev):
    cases = [(N.DT_FP32, N.OP_SUM, 100003), (N.DT_BF16, N.OP_SUM, 1 << 20), (N.DT_INT32, N.OP_PROD, 7),
             (N.DT_FP16, N.OP_MAX, 65537), (N.DT_FP32, N.OP_MIN, 3 << 20), (N.DT_BF16, N.OP_PROD, 1),
             (N.DT_FP32, N.OP_SUM, 0)]
    ring = Ring(dev, capacity=4)                 # 4 slots, 21 triggers: the ring wraps five times
    closed = False
    try:
        with DevBufs(dev) as b:
            total = 0
            for rep in range(3):
                for dtype, op, n in cases:
                    a, c = seeded_inputs(dtype, 2, max(n, 1), seed=rep * 10 + op)
                    da, dc = b.put(a), b.put(c)
                    do = b.alloc(max(n, 1) * 4)
                    idx = ring.enqueue(da, dc, do, n, dtype, op)
                    ring.wait(idx)
                    total += 1
                    if n:
                        got = dev.to_host(do, n, N.NP_DTYPE[dtype])
                        assert_parity(got, O.reduce2(a[:n], c[:n], dtype, op), dtype, op, f"fifo {dtype} {op} {n}")
            # several independent triggers in flight at once, collected afterwards
            a, c = seeded_inputs(N.DT_FP32, 2, 4 * 50000, seed=77)
            da, dc, do = b.put(a), b.put(c), b.alloc(4 * 50000 * 4)
            slots = [ring.enqueue(da + q * 200000, dc + q * 200000, do + q * 200000, 50000, N.DT_FP32, N.OP_SUM)
                     for q in range(4)]
            for s in slots:
                ring.wait(s)
            total += 4
            assert_parity(dev.to_host(do, 200000, np.float32), O.reduce2(a, c, N.DT_FP32, N.OP_SUM), N.DT_FP32, N.OP_SUM)
            # a ring reduce-scatter chain: each step's output is the next step's input1 (output == input1)
            k, n = 5, 300001
            ins = seeded_inputs(N.DT_FP32, k, n, seed=5)
            dins = [b.put(x) for x in ins]
            for p in range(1, k):
                ring.wait(ring.enqueue(dins[0], dins[p], dins[0], n, N.DT_FP32, N.OP_SUM))
                total += 1
            assert_parity(dev.to_host(dins[0], n, np.float32), O.reduce_copy(ins, N.DT_FP32, N.OP_SUM), N.DT_FP32,
                          N.OP_SUM, "chain")
            # an op outside the enum is completed (so the producer is not left waiting) and counted
            ring.wait(ring.enqueue(dins[0], dins[1], dins[0], 16, N.DT_FP32, 7))
            total += 1
            w = ring.words()
            assert w[0] == 4 and w[2] == total                      # capacity, produced
            host = ring.host
            lib.fx_fifo_terminate(host)
            dev.stream_sync(ring.stream)
            assert int(w[1]) == total                               # consumed, published by the kernel on its way out
            reason, done, bad = ring.close()
            closed = True
            assert (reason, done, bad) == (N.SUCCESS + 1, total, 1)  # FX_FIFO_EXIT_TERMINATE
    finally:
        if not closed:
            ring.close()


def test_consumer_ends_by_itself_when_idle(dev):
    """No trigger, no terminate: the poll limit ends the kernel."""
    ring = Ring(dev, capacity=8, poll_limit=2000)
    t0 = time.time()
    dev.stream_sync(ring.stream)
    assert time.time() - t0 < DEADLINE
    reason, done, bad = ring.close()
    assert (reason, done, bad) == (2, 0, 0)                          # FX_FIFO_EXIT_IDLE


def test_triggers_enqueued_before_the_launch_are_served(dev):
    """The consumer starts at the ring's `consumed` index, so what the host put in
    the ring before launching it is executed first."""
    cap, n = 8, 70001
    host = dev.malloc(lib.fx_fifo_bytes(cap), N.MEM_HOST)
    N.check(lib.fx_fifo_init(host, cap))
    a, c = seeded_inputs(N.DT_FP32, 2, n, seed=3)
    with DevBufs(dev) as b:
        da, dc = b.put(a), b.put(c)
        outs = [b.alloc(n * 4) for _ in range(3)]
        idx = C.c_int(-1)
        slots = []
        for o, op in zip(outs[:2], (N.OP_SUM, N.OP_MIN)):            # two triggers wait in the ring
            N.check(lib.fx_fifo_enqueue(host, da, dc, o, n, 32, N.DT_FP32, op, C.byref(idx)))
            assert idx.value >= 0
            slots.append(idx.value)
        dptr = C.c_void_p()
        N.check(dev.t.hostGetDevicePointer(C.byref(dptr), host))
        stream = dev.stream_create()
        cons = C.c_void_p()
        N.check(lib.fx_fifo_consumer_create(C.byref(cons), cap))
        N.check(lib.fx_fifo_consumer_launch(cons, dptr, host, POLL_LIMIT, dev.raw_stream(stream)))
        N.check(lib.fx_fifo_enqueue(host, da, dc, outs[2], n, 32, N.DT_FP32, N.OP_MAX, C.byref(idx)))   # and one after
        slots.append(idx.value)
        t0 = time.time()
        try:
            for s in slots:
                while lib.fx_fifo_poll_state(host, s) != COMPLETE:
                    assert time.time() - t0 < DEADLINE, "a trigger enqueued before the launch was never served"
                N.check(lib.fx_fifo_set_state(host, s, AVAILABLE))
        finally:
            lib.fx_fifo_terminate(host)
            dev.stream_sync(stream)
        for o, op in zip(outs, (N.OP_SUM, N.OP_MIN, N.OP_MAX)):
            assert_parity(dev.to_host(o, n, np.float32), O.reduce2(a, c, N.DT_FP32, op), N.DT_FP32, op, f"op {op}")
        reason, done, bad = C.c_int(-1), C.c_uint64(), C.c_uint64()
        N.check(lib.fx_fifo_consumer_status(cons, C.byref(reason), C.byref(done), C.byref(bad)))
        assert (reason.value, done.value, bad.value) == (1, 3, 0)
        lib.fx_fifo_consumer_destroy(cons)
        dev.stream_destroy(stream)
    dev.free(host, N.MEM_HOST)


def test_second_launch_does_not_repeat_a_trigger_that_was_running_at_terminate(dev):
    """terminate right behind a large in-place trigger: the consumer leaves only
    after that trigger is complete and `consumed` says so, so a second consumer
    on the same ring starts behind it (a repeat would add input 2 twice)."""
    cap, n = 4, 24 << 20
    host = dev.malloc(lib.fx_fifo_bytes(cap), N.MEM_HOST)
    N.check(lib.fx_fifo_init(host, cap))
    words = np.ctypeslib.as_array(C.cast(host, C.POINTER(C.c_uint64)), shape=(4,))
    a, c = seeded_inputs(N.DT_FP32, 2, n, seed=21)
    small = seeded_inputs(N.DT_INT32, 2, 1000, seed=22)
    with DevBufs(dev) as b:
        da, dc = b.put(a), b.put(c)
        ds0, ds1, dso = b.put(small[0]), b.put(small[1]), b.alloc(4000)
        dptr = C.c_void_p()
        N.check(dev.t.hostGetDevicePointer(C.byref(dptr), host))
        stream = dev.stream_create()
        cons = C.c_void_p()
        N.check(lib.fx_fifo_consumer_create(C.byref(cons), cap))
        idx = C.c_int(-1)
        try:
            N.check(lib.fx_fifo_consumer_launch(cons, dptr, host, POLL_LIMIT, dev.raw_stream(stream)))
            N.check(lib.fx_fifo_enqueue(host, da, dc, da, n, 32, N.DT_FP32, N.OP_SUM, C.byref(idx)))   # a += c
            assert idx.value == 0
        finally:
            lib.fx_fifo_terminate(host)                               # without waiting for Complete
            dev.stream_sync(stream)
        assert lib.fx_fifo_poll_state(host, 0) == COMPLETE
        assert int(words[1]) == int(words[2]) == 1                    # consumed == produced
        N.check(lib.fx_fifo_set_state(host, 0, AVAILABLE))
        words[3] = 0                                                  # same ring, new session
        try:
            N.check(lib.fx_fifo_consumer_launch(cons, dptr, host, POLL_LIMIT, dev.raw_stream(stream)))
            N.check(lib.fx_fifo_enqueue(host, ds0, ds1, dso, 1000, 32, N.DT_INT32, N.OP_MAX, C.byref(idx)))
            assert idx.value == 1
            t0 = time.time()
            while lib.fx_fifo_poll_state(host, 1) != COMPLETE:
                assert time.time() - t0 < DEADLINE, "second session's trigger never completed"
        finally:
            lib.fx_fifo_terminate(host)
            dev.stream_sync(stream)
        assert_parity(dev.to_host(da, n, np.float32), O.reduce2(a, c, N.DT_FP32, N.OP_SUM), N.DT_FP32, N.OP_SUM, "once")
        assert_parity(dev.to_host(dso, 1000, np.int32), O.reduce2(small[0], small[1], N.DT_INT32, N.OP_MAX), N.DT_INT32,
                      N.OP_MAX, "second session")
        reason, done, bad = C.c_int(-1), C.c_uint64(), C.c_uint64()
        N.check(lib.fx_fifo_consumer_status(cons, C.byref(reason), C.byref(done), C.byref(bad)))
        assert (reason.value, done.value, bad.value) == (1, 1, 0)     # the second session completed one trigger
        lib.fx_fifo_consumer_destroy(cons)
        dev.stream_destroy(stream)
    dev.free(host, N.MEM_HOST)


def test_batch_of_independent_triggers_through_the_producer_loop(dev):
    """fx_fifo_run_batch: 300 independent triggers of mixed sizes, types and ops
    through a 16-slot ring (the ring wraps 18 times, many triggers in flight at
    once, workgroups inspect them in batches); every output against the oracle.
    With no consumer running the loop gives up instead of spinning for ever."""
    cap, total = 16, 300
    ring = Ring(dev, cap)
    closed = False
    try:
        rng = np.random.default_rng(9)
        kinds = [(N.DT_FP32, N.OP_SUM), (N.DT_BF16, N.OP_MAX), (N.DT_INT32, N.OP_PROD), (N.DT_UINT8, N.OP_MIN),
                 (N.DT_FP64, N.OP_SUM), (N.DT_FP16, N.OP_AVG)]
        with DevBufs(dev) as b:
            trig = (N.ReduceTrigger * total)()
            cases = []
            for i in range(total):
                dtype, op = kinds[i % len(kinds)]
                n = int(rng.choice([1, 7, 1000, 4096, 70001, 300000]))
                a, c = seeded_inputs(dtype, 2, n, seed=1000 + i)
                da, dc, do = b.put(a), b.put(c), b.alloc(n * N.DTYPE_SIZE[dtype])
                lib.fx_trigger_set(C.byref(trig[i]), da, dc, do, n, 32, dtype, op, ENQUEUED)
                cases.append((dtype, op, n, a, c, do))
            N.check(lib.fx_fifo_run_batch(ring.host, trig, total, 200_000_000))
            assert int(ring.words()[2]) == total                       # produced
            reason, done, bad = ring.close()                           # before the slow checking: the consumer would idle out
            closed = True
            assert (reason, done, bad) == (1, total, 0)
            for i, (dtype, op, n, a, c, do) in enumerate(cases):
                assert_parity(dev.to_host(do, n, N.NP_DTYPE[dtype]), O.reduce2(a, c, dtype, op), dtype, op, f"trigger {i}")
    finally:
        if not closed:
            ring.close()
    # no consumer: nothing ever completes, the producer loop reports it
    host = dev.malloc(lib.fx_fifo_bytes(4), N.MEM_HOST)
    N.check(lib.fx_fifo_init(host, 4))
    one = (N.ReduceTrigger * 1)()
    lib.fx_trigger_set(C.byref(one[0]), 4096, 8192, 12288, 0, 32, N.DT_FP32, N.OP_SUM, ENQUEUED)
    assert lib.fx_fifo_run_batch(host, one, 1, 1000) == N.INTERNAL_ERROR
    assert lib.fx_fifo_run_batch(None, one, 1, 1000) == N.INVALID_ARGUMENT
    dev.free(host, N.MEM_HOST)


def test_long_chain_of_dependent_triggers_sees_every_previous_result(dev):
    """acc = acc + x_i forty times over 3 Mi elements (every workgroup of every die
    takes part in each trigger, and trigger i + 1 reads what trigger i wrote, most of
    it from another die): the results are stored through the caches and the next
    trigger's workgroups invalidate before they load, so nothing stale is read."""
    n, steps = 3 << 20, 40
    ring = Ring(dev, capacity=8)
    closed = False
    try:
        rng = np.random.default_rng(31)
        acc = rng.integers(-1000, 1000, n).astype(np.int32)
        xs = [rng.integers(-1000, 1000, n).astype(np.int32) for _ in range(4)]
        with DevBufs(dev) as b:
            dacc = b.put(acc)
            dxs = [b.put(x) for x in xs]
            want = acc.copy()
            for i in range(steps):
                ring.wait(ring.enqueue(dacc, dxs[i % 4], dacc, n, N.DT_INT32, N.OP_SUM))      # output == input 1
                want += xs[i % 4]
            # ping-pong between two buffers, max: a stale read would let an old, smaller value survive
            da, db2 = b.put(acc), b.alloc(n * 4)
            hi = acc.copy()
            for i in range(steps):
                src, dst = (da, db2) if i % 2 == 0 else (db2, da)
                ring.wait(ring.enqueue(src, dxs[i % 4], dst, n, N.DT_INT32, N.OP_MAX))
                hi = np.maximum(hi, xs[i % 4])
            reason, done, bad = ring.close()
            closed = True
            assert (reason, done, bad) == (1, 2 * steps, 0)
            assert np.array_equal(dev.to_host(dacc, n, np.int32), want)
            assert np.array_equal(dev.to_host(da, n, np.int32), hi)
    finally:
        if not closed:
            ring.close()


def test_in_order_consumer_runs_dependent_triggers_enqueued_back_to_back(dev, monkeypatch):
    """FX_FIFO_IN_ORDER=1: the reference consumer's serial semantics
    (flagcx_reduce_kernel_device.cu:104-185).  Sixty triggers, each reading what
    the one before it wrote, are pushed through a 16-slot ring by the producer
    loop without waiting for any of them in between; sizes alternate between one
    tile and every workgroup of every die.  A consumer that let two of them run
    side by side, or read a stale line, would not reproduce the sequential result."""
    monkeypatch.setenv("FX_FIFO_IN_ORDER", "1")
    ring = Ring(dev, capacity=16)
    monkeypatch.delenv("FX_FIFO_IN_ORDER")
    closed = False
    try:
        rng = np.random.default_rng(77)
        n, steps = 3 << 20, 60
        acc = rng.integers(-1000, 1000, n).astype(np.int32)
        xs = [rng.integers(-1000, 1000, n).astype(np.int32) for _ in range(3)]
        with DevBufs(dev) as b:
            dacc, dalt = b.put(acc), b.put(np.zeros(n, np.int32))     # (no memset / device-wide wait while the consumer runs)
            dxs = [b.put(x) for x in xs]
            trig = (N.ReduceTrigger * steps)()
            want, other = acc.copy(), np.zeros(n, np.int32)
            src, dst, hsrc, hdst = dacc, dalt, want, other
            for i in range(steps):
                cnt = n if i % 3 else 4096 + i            # a short trigger in between: only its first elements move on
                op = N.OP_SUM if i % 2 else N.OP_MAX
                lib.fx_trigger_set(C.byref(trig[i]), src, dxs[i % 3], dst, cnt, 32, N.DT_INT32, op, ENQUEUED)
                hdst[:cnt] = (hsrc[:cnt] + xs[i % 3][:cnt]) if op == N.OP_SUM else np.maximum(hsrc[:cnt], xs[i % 3][:cnt])
                src, dst, hsrc, hdst = dst, src, hdst, hsrc     # ping-pong: the next one reads what this one wrote
            N.check(lib.fx_fifo_run_batch(ring.host, trig, steps, 400_000_000))
            reason, done, bad = ring.close()
            closed = True
            assert (reason, done, bad) == (1, steps, 0)
            got = {dacc: dev.to_host(dacc, n, np.int32), dalt: dev.to_host(dalt, n, np.int32)}
            assert np.array_equal(got[src], hsrc), "last trigger's output differs from the sequential result"
            assert np.array_equal(got[dst], hdst), "the other buffer (second-to-last output) differs"
    finally:
        if not closed:
            ring.close()


def test_ring_allreduce_driven_through_the_fifo(dev):
    """What an unmodified uniRunner does with this consumer behind its FIFO
    (uni_runner_impl.cc:661-1007): n-1 reduce-scatter steps whose reduce nodes --
    one per rank, slice and red-slice: in1 = the previous rank's partial, in2 = own
    data, out = own receive buffer -- go through the ring as triggers, each step
    waiting for the one before; then the all-gather copies.  fp32, so the result
    must equal the hop-by-hop ring oracle bit for bit."""
    from flagcx_amd import kernels as K
    n, count, nslices, nred = 8, 8 * 50021 + 5, 2, 3
    dtype, es = N.DT_FP32, 4
    sends = seeded_inputs(dtype, n, count, seed=41)
    rng = np.random.default_rng(41)
    sends = [(a * 10.0 ** rng.integers(-3, 9, count)).astype(np.float32) for a in sends]     # make the order matter
    want = O.ring_allreduce(sends, dtype, N.OP_SUM)
    ring = Ring(dev, capacity=128)
    closed = False
    try:
        with DevBufs(dev) as b:
            ds = [b.put(a) for a in sends]
            dr = [b.alloc(count * es) for _ in range(n)]
            ntrig = 0
            for i in range(n - 1):                                   # reduce-scatter steps
                trig = (N.ReduceTrigger * (n * nslices * nred))()
                t = 0
                for r in range(n):
                    prev, rx = (r - 1) % n, (r - i - 1) % n
                    ccnt, coff = K.split(count, n, rx)
                    partial = ds[prev] if i == 0 else dr[prev]
                    for s in range(nslices):
                        scnt, soff = K.split(ccnt, nslices, s)
                        for q in range(nred):
                            rcnt, roff = K.split(scnt, nred, q)
                            off = (coff + soff + roff) * es
                            lib.fx_trigger_set(C.byref(trig[t]), partial + off, ds[r] + off, dr[r] + off, rcnt, 32, dtype,
                                               N.OP_SUM, ENQUEUED)
                            t += 1
                N.check(lib.fx_fifo_run_batch(ring.host, trig, t, 200_000_000))
                ntrig += t
            reason, done, bad = ring.close()
            closed = True
            assert (reason, done, bad) == (1, ntrig, 0)
            stream = dev.stream_create()
            for i in range(n - 1):                                   # all-gather steps: chunk (r - i) % n from the previous rank
                copies = []
                for r in range(n):
                    ccnt, coff = K.split(count, n, (r - i) % n)
                    copies.append((dr[(r - 1) % n] + coff * es, dr[r] + coff * es, ccnt * es))
                N.check(K.copy_slices(copies, dev.raw_stream(stream)))
            dev.stream_sync(stream)
            dev.stream_destroy(stream)
            for r in range(n):
                got = dev.to_host(dr[r], count, np.float32)
                assert np.array_equal(got.view(np.uint32), want[r].view(np.uint32)), f"rank {r}"
    finally:
        if not closed:
            ring.close()
