"""GPU parity of the batched slice kernels (k-way descriptors, the reference's
2-input triggers, device-resident plans), the copy phase and alltoallv
pack / unpack, against the CPU oracle."""
import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from oracle import fx_oracle as O
from tests.util import DTYPES, OPS, DevBufs, assert_parity, is_nan16, seeded_inputs

pytestmark = pytest.mark.gpu


def _ragged_slices(rng, total, nslices):
    """Non-overlapping (offset, count) pieces of [0,total) with gaps, odd sizes and an empty one."""
    cuts = np.sort(rng.choice(np.arange(1, total), size=2 * nslices - 1, replace=False))
    bounds = np.concatenate([[0], cuts, [total]])
    sl = [(int(bounds[2 * i]), int(bounds[2 * i + 1] - bounds[2 * i])) for i in range(nslices)]
    sl.insert(len(sl) // 2, (sl[0][0], 0))
    return sl


@pytest.mark.parametrize("dname", list(DTYPES))
@pytest.mark.parametrize("k", [1, 2, 5, 8])
def test_reduce_slices_ragged(dev, dname, k):
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    rng = np.random.default_rng(k)
    total = 400000
    ins = seeded_inputs(dtype, k, total, seed=21)
    for nsl, op in ((3, N.OP_SUM), (40, N.OP_MAX), (70, N.OP_PROD), (5, N.OP_MIN)):   # 40, 70 > one argument block
        sl = _ragged_slices(rng, total, nsl)
        with DevBufs(dev) as b:
            dins = [b.put(a) for a in ins]
            dout = b.alloc(total * es)
            dev.memset(dout, 0x5A, total * es)
            descs = [([p + o * es for p in dins], dout + o * es, c) for o, c in sl]
            N.check(K.reduce_slices(descs, k, dtype, op), "fx_reduce_slices")
            dev.sync()
            got = dev.to_host(dout, total, N.NP_DTYPE[dtype])
        want = np.frombuffer(bytes([0x5A]) * (total * es), dtype=N.NP_DTYPE[dtype]).copy()
        for o, c in sl:
            if c:
                want[o:o + c] = O.reduce_copy([a[o:o + c] for a in ins], dtype, op)
        assert_parity(got, want, dtype, op, f"slices {dname} k={k} n={nsl}")


def test_plan_equals_inline_slices_and_is_relaunchable(dev):
    dtype, op, k, total = N.DT_BF16, N.OP_SUM, 8, 600000
    rng = np.random.default_rng(3)
    ins = seeded_inputs(dtype, k, total, seed=1)
    sl = _ragged_slices(rng, total, 50)
    with DevBufs(dev) as b:
        dins = [b.put(a) for a in ins]
        dout = b.alloc(total * 2)
        descs = [([p + o * 2 for p in dins], dout + o * 2, c) for o, c in sl]
        plan = K.Plan(descs, k, dtype, op)
        for _ in range(3):
            dev.memset(dout, 0, total * 2)
            N.check(plan.launch(), "fx_plan_launch")
            dev.sync()
            got = dev.to_host(dout, total, np.uint16)
            want = np.zeros(total, np.uint16)
            for o, c in sl:
                if c:
                    want[o:o + c] = O.reduce_copy([a[o:o + c] for a in ins], dtype, op)
            assert_parity(got, want, dtype, op, "plan")
        plan.destroy()
        empty = K.Plan([], 2, dtype, op)
        assert empty.launch() == N.SUCCESS
        empty.destroy()


def test_triggers_ring_step_semantics(dev):
    """2-input triggers in the reference's 32-byte format, output aliasing input1
    (ring: output == input1, uni_runner_impl.cc:864-878), mixed dtype/op runs."""
    n = 70001
    f = seeded_inputs(N.DT_FP32, 2, n, seed=2)
    i = seeded_inputs(N.DT_INT32, 2, n, seed=3)
    h = seeded_inputs(N.DT_FP16, 2, n, seed=4)
    with DevBufs(dev) as b:
        df, di, dh = [b.put(a) for a in f], [b.put(a) for a in i], [b.put(a) for a in h]
        half = n // 2
        trig = [
            K.make_trigger(df[0], df[1], df[0], half, 32, N.DT_FP32, N.OP_SUM),                      # in place on in1
            K.make_trigger(df[0] + half * 4, df[1] + half * 4, df[0] + half * 4, n - half, 32, N.DT_FP32, N.OP_SUM),
            K.make_trigger(di[0], di[1], di[0], n, 32, N.DT_INT32, N.OP_PROD),
            K.make_trigger(dh[0], dh[1], dh[0], n, 32, N.DT_FP16, N.OP_MAX),
            K.make_trigger(dh[0], dh[1], dh[1], 0, 32, N.DT_FP16, N.OP_MAX),                         # empty
        ]
        N.check(K.reduce_triggers(trig), "fx_reduce_triggers")
        dev.sync()
        assert_parity(dev.to_host(df[0], n, np.float32), O.reduce2(f[0], f[1], N.DT_FP32, N.OP_SUM), N.DT_FP32, N.OP_SUM)
        assert_parity(dev.to_host(di[0], n, np.int32), O.reduce2(i[0], i[1], N.DT_INT32, N.OP_PROD), N.DT_INT32,
                      N.OP_PROD)
        assert_parity(dev.to_host(dh[0], n, np.uint16), O.reduce2(h[0], h[1], N.DT_FP16, N.OP_MAX), N.DT_FP16, N.OP_MAX)
        bad = [K.make_trigger(df[0], df[1], df[0], 4, 32, N.DT_FP32, 7)]
        assert K.reduce_triggers(bad) == N.INVALID_ARGUMENT


def test_reduce2_all_types(dev):
    for dname, dtype in DTYPES.items():
        a, c = seeded_inputs(dtype, 2, 12345, seed=9)
        for op in OPS.values():
            with DevBufs(dev) as b:
                da, dc, do = b.put(a), b.put(c), b.alloc(12345 * N.DTYPE_SIZE[dtype])
                N.check(K.reduce2(do, da, dc, 12345, dtype, op), "fx_reduce2")
                dev.sync()
                got = dev.to_host(do, 12345, N.NP_DTYPE[dtype])
            assert_parity(got, O.reduce2(a, c, dtype, op), dtype, op, f"reduce2 {dname} {op}")


def test_copy_slices_byte_granular(dev):
    rng = np.random.default_rng(12)
    src = rng.integers(0, 256, 3_000_000, dtype=np.uint8)
    # (src offset, dst offset, bytes): aligned, co-misaligned, differently misaligned, odd lengths, tiny, empty
    cases = [(0, 0, 1 << 20), (1 << 20, (1 << 20) + 16, 65536), (1200003, 1300003, 70001), (1400001, 1500006, 33333),
             (1600000, 1700002, 2), (1800001, 1800001 + 100000, 1), (5, 2000000, 0), (2100002, 2200004, 40000)]
    with DevBufs(dev) as b:
        dsrc = b.put(src)
        ddst = b.alloc(src.size)
        dev.memset(ddst, 0xEE, src.size)
        N.check(K.copy_slices([(dsrc + s, ddst + d, n) for s, d, n in cases]), "fx_copy_slices")
        dev.sync()
        got = dev.to_host(ddst, src.size, np.uint8)
    want = np.full(src.size, 0xEE, np.uint8)
    for s, d, n in cases:
        want[d:d + n] = src[s:s + n]
    assert np.array_equal(got, want)


def test_long_copies_at_every_kind_of_line_phase(dev):
    """Copies long enough for the striped hand-out (4 MiB and more) whose source sits
    at the destination's offset within a 128-byte line, at another 16-byte multiple,
    or at an odd byte: several to a launch, so that later ones start at a tile number
    that is not a multiple of eight, through fx_copy_slices, fx_pack / fx_unpack and the
    one-input fx_reduce_copy.  Bytes either side of every destination stay untouched."""
    rng = np.random.default_rng(77)
    mib = 1 << 20
    src = rng.integers(0, 256, 40 * mib, dtype=np.uint8)
    # (src offset, dst offset, bytes)
    cases = [(0, 0, 5 * mib), (5 * mib + 16, 5 * mib + 64, 4 * mib + 4096), (10 * mib + 48, 10 * mib, 6 * mib + 17),
             (17 * mib + 1, 17 * mib + 128, 4 * mib + 1), (22 * mib + 64, 22 * mib + 64, 4 * mib),
             (27 * mib + 100, 27 * mib + 36, 7 * mib - 5), (35 * mib, 35 * mib + 2, 4 * mib + 300)]
    with DevBufs(dev) as b:
        dsrc = b.put(src)
        ddst = b.alloc(src.size)
        for order in (cases, cases[::-1], cases[3:4]):
            dev.memset(ddst, 0xEE, src.size)
            N.check(K.copy_slices([(dsrc + s, ddst + d, n) for s, d, n in order]), "fx_copy_slices")
            dev.sync()
            got = dev.to_host(ddst, src.size, np.uint8)
            want = np.full(src.size, 0xEE, np.uint8)
            for s, d, n in order:
                want[d:d + n] = src[s:s + n]
            assert np.array_equal(got, want)
        # the same through the typed one-input reduce-copy (fp32: element offsets 0..31 cover every 16-byte phase and
        # the element-misaligned ones) and through pack / unpack with element displacements
        s32 = src.view(np.uint32)
        for so, do, n in ((3, 0, 5 * mib // 4), (4, 8, 4 * mib // 4 + 1), (0, 17, 6 * mib // 4 + 3), (12, 28, 4 * mib // 4)):
            dev.memset(ddst, 0xEE, src.size)
            N.check(K.reduce_copy(ddst + 4 * do, [dsrc + 4 * so], n, N.DT_FP32, N.OP_SUM, 0), "fx_reduce_copy k=1")
            dev.sync()
            got = dev.to_host(ddst, n + do + 64, np.uint32)
            assert np.array_equal(got[do:do + n], s32[so:so + n]), (so, do, n)
            assert (got[:do] == 0xEEEEEEEE).all() and (got[do + n:] == 0xEEEEEEEE).all(), (so, do, n)
        counts = [mib + 3, 0, 2 * mib, mib // 2, mib + 1, 3 * mib // 2]          # fp32 elements: 4-8 MiB segments and a short one
        sdispls, pos = [], 5
        for c in counts:
            sdispls.append(pos)
            pos += c + 3
        total = sum(counts)
        dpacked = b.alloc(total * 4 + 64)
        dev.memset(dpacked, 0x77, total * 4 + 64)
        N.check(K.pack(dpacked, dsrc, counts, sdispls, N.DT_FP32), "fx_pack")
        dev.memset(ddst, 0xEE, src.size)
        rdispls = [d + 7 for d in sdispls]
        N.check(K.unpack(ddst, dpacked, counts, rdispls, N.DT_FP32), "fx_unpack")
        dev.sync()
        packed = dev.to_host(dpacked, total + 16, np.uint32)
        back = dev.to_host(ddst, pos + 64, np.uint32)
    assert np.array_equal(packed[:total], O.pack(s32, counts, sdispls))
    assert (packed[total:] == 0x77777777).all()
    want = O.unpack(np.full(pos + 64, 0xEEEEEEEE, np.uint32), packed[:total], counts, rdispls)
    assert np.array_equal(back, want)


@pytest.mark.parametrize("dname", ["bf16", "fp32", "int32", "uint8", "fp64"])
def test_reduce_bcast_many_inputs_many_outputs(dev, dname):
    """fx_reduce_bcast: one segment, up to 64 inputs folded once (starting at
    `first`) and stored to up to 64 outputs -- more ranks than a slice descriptor
    has slots.  Odd lengths, buffers off 16-byte alignment (alike, and one output
    at its own offset: the reduce-plus-copies route), a segment long enough for the
    striped hand-out, in place; nothing written outside any output."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    npdt = N.NP_DTYPE[dtype]
    rng = np.random.default_rng(es)
    ve = 16 // es
    cases = [(9, 9, 40001, 0, 0), (17, 3, 1, 2, 0), (12, 16, 65536 + 5, 5, 3), (1, 12, 300007, 0, 1), (33, 33, 2048, 7, 0),
             (64, 64, 1500, 63, 2), (10, 2, (5 << 20) // es + 3, 4, 0)]
    for k, nout, n, first, mis in cases:
        for op in (N.OP_SUM, N.OP_MAX) if k < 30 else (N.OP_SUM,):
            ins = seeded_inputs(dtype, k, n, seed=k * 100 + nout)
            want = O.reduce_copy(ins, dtype, op, first=first)
            for odd_one in (False, True):
                with DevBufs(dev) as b:
                    dins = [b.put(a, pad_before=mis * es) for a in ins]
                    outs = []
                    for o in range(nout):
                        lead = (mis + (1 if odd_one and o == nout - 1 and ve > 1 else 0)) * es
                        base = b.alloc(lead + n * es + 64)
                        dev.memset(base, 0xA5, lead + n * es + 64)
                        outs.append(base + lead)
                    N.check(K.reduce_bcast(outs, dins, n, dtype, op, first), f"fx_reduce_bcast k={k} nout={nout}")
                    dev.sync()
                    for o, d in enumerate(outs):
                        assert_parity(dev.to_host(d, n, npdt), want, dtype, op, f"{dname} k={k} nout={nout} n={n} out {o}")
                        assert (dev.to_host(d + n * es, 32, np.uint8) == 0xA5).all(), "wrote past an output"
                        lead = d % 16
                        if lead:
                            assert (dev.to_host(d - lead, lead, np.uint8) == 0xA5).all(), "wrote before an output"
    # in place on every rank's buffer (the all-reduce shape), and a broadcast copy
    k = 11
    ins = seeded_inputs(dtype, k, 77777, seed=3)
    want = O.reduce_copy(ins, dtype, N.OP_SUM)
    with DevBufs(dev) as b:
        dins = [b.put(a) for a in ins]
        N.check(K.reduce_bcast(dins, dins, 77777, dtype, N.OP_SUM), "in place")
        dev.sync()
        for d in dins:
            assert_parity(dev.to_host(d, 77777, npdt), want, dtype, N.OP_SUM, f"{dname} in place")
        outs = [b.alloc(77777 * es + 8) + (o % 2) for o in range(13)]          # odd byte offsets: the copy granularity adapts
        N.check(K.reduce_bcast(outs, [dins[0] + es], (77777 - 1) * es, dtype, -1), "broadcast copy")
        dev.sync()
        src = dev.to_host(dins[0] + es, (77777 - 1) * es, np.uint8)
        for d in outs:
            assert np.array_equal(dev.to_host(d, (77777 - 1) * es, np.uint8), src)
    assert K.reduce_bcast([1], [], 4, dtype, N.OP_SUM) == N.INVALID_ARGUMENT
    assert K.reduce_bcast([16] * 65, [16], 4, dtype, N.OP_SUM) == N.INVALID_ARGUMENT
    assert K.reduce_bcast([16], [16, 16], 4, dtype, N.OP_SUM, first=2) == N.INVALID_ARGUMENT
    assert K.reduce_bcast([16], [16, 16], 4, dtype, -1) == N.INVALID_ARGUMENT


@pytest.mark.parametrize("dname", ["bf16", "fp32", "int64", "uint8"])
def test_reduce_chunks_is_a_collective_over_many_ranks_in_one_launch(dev, dname):
    """fx_reduce_chunks with the three shapes it exists for, 12 and 17 ranks:
    a ring-order all-reduce (chunk c folded from rank c on, stored to every rank),
    a reduce-scatter (chunk r of every send buffer folded onto rank r alone) and an
    all-gather (rank q's block copied into slot q of every rank), each in one call,
    with ragged chunk sizes, an empty chunk and buffers off 16-byte alignment."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    npdt = N.NP_DTYPE[dtype]
    for n, count, mis in ((12, 100003, 0), (17, 40000, 3), (9, 5, 1), (64, 6400, 0)):
        sends = seeded_inputs(dtype, n, count, seed=n)
        base, rem = divmod(count, n)
        cnt = [base + (c < rem) for c in range(n)]
        off = [c * base + min(c, rem) for c in range(n)]
        with DevBufs(dev) as b:
            ds = [b.put(a, pad_before=mis * es) for a in sends]
            lead = mis * es
            raw = [b.alloc(lead + count * es + 64) for _ in range(n)]
            for q in raw:
                dev.memset(q, 0xA5, lead + count * es + 64)
            dr = [q + lead for q in raw]
            # ring-order all-reduce
            ch = [(off[c], off[c], cnt[c], c, -1, -1) for c in range(n)]
            N.check(K.reduce_chunks(dr, ds, ch, dtype, N.OP_SUM), "all-reduce chunks")
            dev.sync()
            want = np.empty(count, npdt)
            for c in range(n):
                want[off[c]:off[c] + cnt[c]] = O.reduce_copy([a[off[c]:off[c] + cnt[c]] for a in sends], dtype, N.OP_SUM,
                                                             first=c) if cnt[c] else []
            for r in range(n):
                assert_parity(dev.to_host(dr[r], count, npdt), want, dtype, N.OP_SUM, f"{dname} n={n} all-reduce rank {r}")
                assert (dev.to_host(dr[r] + count * es, 32, np.uint8) == 0xA5).all()
                if lead:
                    assert (dev.to_host(raw[r], lead, np.uint8) == 0xA5).all()
            # reduce-scatter: chunk r -> rank r, at the start of its buffer
            for q in raw:
                dev.memset(q, 0xA5, lead + count * es + 64)
            ch = [(off[r], 0, cnt[r], (r + 1) % n, -1, r) for r in range(n)]
            N.check(K.reduce_chunks(dr, ds, ch, dtype, N.OP_MAX), "reduce-scatter chunks")
            dev.sync()
            for r in range(n):
                if cnt[r]:
                    w = O.reduce_copy([a[off[r]:off[r] + cnt[r]] for a in sends], dtype, N.OP_MAX, first=(r + 1) % n)
                    assert_parity(dev.to_host(dr[r], cnt[r], npdt), w, dtype, N.OP_MAX, f"{dname} n={n} reduce-scatter rank {r}")
                assert (dev.to_host(dr[r] + cnt[r] * es, 32, np.uint8) == 0xA5).all(), "wrote past a reduce-scatter chunk"
            # all-gather as a copy: block q of `blk` bytes from rank q into slot q of every rank
            blk = (count // n) * es
            if blk:
                for q in raw:
                    dev.memset(q, 0xA5, lead + count * es + 64)
                ch = [(0, q * blk, blk, 0, q, -1) for q in range(n)]
                N.check(K.reduce_chunks(dr, ds, ch, dtype, -1), "all-gather chunks")
                dev.sync()
                want8 = np.concatenate([a.view(np.uint8)[:blk] for a in sends])
                for r in range(n):
                    assert np.array_equal(dev.to_host(dr[r], n * blk, np.uint8), want8), f"all-gather rank {r}"
                    assert (dev.to_host(dr[r] + n * blk, 16, np.uint8) == 0xA5).all()
    with DevBufs(dev) as b:
        p = b.alloc(64)
        assert K.reduce_chunks([p], [p], [(0, 0, 4, 1, -1, -1)], dtype, N.OP_SUM) == N.INVALID_ARGUMENT     # first >= k
        assert K.reduce_chunks([p], [p], [(0, 0, 4, 0, -1, 1)], dtype, N.OP_SUM) == N.INVALID_ARGUMENT      # out_sel >= nout
        assert K.reduce_chunks([p], [p], [(0, 0, 4, 0, -1, -1)], dtype, -1) == N.INVALID_ARGUMENT           # a copy names its input
        assert K.reduce_chunks([p, p + 4], [p], [(0, 0, 1, 0, -1, -1)], N.DT_UINT8, N.OP_SUM) == N.INVALID_ARGUMENT
        assert K.reduce_chunks([p], [p], [], dtype, N.OP_SUM) == N.SUCCESS


def _random_layout(rng, counts, slack):
    """Random non-overlapping displacements for the given segment counts."""
    order = rng.permutation(len(counts))
    displs, pos = [0] * len(counts), 0
    for i in order:
        pos += int(rng.integers(0, slack))
        displs[i] = pos
        pos += int(counts[i])
    return displs, pos + int(rng.integers(0, slack))


@pytest.mark.parametrize("dname,np_t", [("fp32", np.uint32), ("bf16", np.uint16)])
def test_pack_unpack_random_displacements(dev, dname, np_t):
    dtype = DTYPES[dname]
    rng = np.random.default_rng(31)
    for trial in range(4):
        npeers = [8, 8, 3, 40][trial]
        counts = [int(np.exp(rng.uniform(0, np.log(200000)))) for _ in range(npeers)]
        counts[rng.integers(0, npeers)] = 0                       # a silent peer
        if trial == 1:
            counts = [c // 4 * 4 for c in counts]                 # 16-byte friendly segments
        sdispls, slen = _random_layout(rng, counts, 9)
        rdispls, rlen = _random_layout(rng, counts, 9)
        send = rng.integers(0, np.iinfo(np_t).max, slen, dtype=np.uint64).astype(np_t)
        total = sum(counts)
        with DevBufs(dev) as b:
            dsend = b.put(send)
            dpacked = b.alloc(total * send.itemsize + 64)
            drecv = b.alloc(rlen * send.itemsize)
            dev.memset(dpacked, 0x77, total * send.itemsize + 64)
            dev.memset(drecv, 0, rlen * send.itemsize)
            N.check(K.pack(dpacked, dsend, counts, sdispls, dtype), "fx_pack")
            N.check(K.unpack(drecv, dpacked, counts, rdispls, dtype), "fx_unpack")
            dev.sync()
            packed = dev.to_host(dpacked, total, np_t)
            guard = dev.to_host(dpacked + total * send.itemsize, 64, np.uint8)
            recv = dev.to_host(drecv, rlen, np_t)
        assert np.array_equal(packed, O.pack(send, counts, sdispls))
        assert (guard == 0x77).all()
        assert np.array_equal(recv, O.unpack(np.zeros(rlen, np_t), O.pack(send, counts, sdispls), counts, rdispls))
        for c, sd, rd in zip(counts, sdispls, rdispls):           # the identity, segment by segment
            assert np.array_equal(recv[rd:rd + c], send[sd:sd + c])


@pytest.mark.parametrize("dname", ["bf16", "fp32", "int8", "fp64"])
def test_reduce_to_several_outputs_at_once(dev, dname):
    """fx_reduce_bcast_slices: every output equals the oracle's fold; covers 1..8
    outputs, in-place outputs (out[j] == in[j]), odd lengths, unaligned but
    co-aligned buffers, outputs of differing alignment (reduce + copy fallback),
    several slices per launch and more slices than one launch carries."""
    dtype = DTYPES[dname]
    es = N.DTYPE_SIZE[dtype]
    npdt = N.NP_DTYPE[dtype]
    for k, nout, n, off_el, inplace in [(8, 8, 300001, 0, True), (2, 3, 5, 0, False), (3, 1, 70001, 1, False),
                                        (4, 8, (1 << 20) + 3, 3, False), (8, 2, 4 << 20, 0, False),
                                        (5, 4, 1000, None, False)]:
        ins = seeded_inputs(dtype, k, n, seed=k * 10 + nout)
        for op in (N.OP_SUM, N.OP_MIN):
            want = O.reduce_copy(ins, dtype, op)
            with DevBufs(dev) as b:
                pad = (off_el or 0) * es
                dins = [b.put(a, pad_before=pad) for a in ins]
                if inplace:
                    douts = dins[:nout]
                elif off_el is None:            # each output at its own misalignment
                    douts = [b.alloc(n * es + 64) + (j % (16 // es)) * es for j in range(nout)]
                else:
                    douts = [b.alloc(n * es + pad + 64) + pad for _ in range(nout)]
                N.check(K.reduce_bcast_slices([(dins, douts, n)], k, nout, dtype, op), "fx_reduce_bcast_slices")
                dev.sync()
                for j, d in enumerate(douts):
                    assert_parity(dev.to_host(d, n, npdt), want, dtype, op, f"{dname} k={k} nout={nout} n={n} out {j}")
    # 40 slices of uneven length cut from one pair of buffers, three outputs, one call
    k, nout, total = 2, 3, 500000
    ins = seeded_inputs(dtype, k, total, seed=3)
    want = O.reduce_copy(ins, dtype, N.OP_SUM)
    cuts = np.unique(np.random.default_rng(5).integers(0, total, 39))
    edges = [0] + cuts.tolist() + [total]
    with DevBufs(dev) as b:
        dins = [b.put(a) for a in ins]
        douts = [b.alloc(total * es) for _ in range(nout)]
        for d in douts:
            dev.memset(d, 0x5A, total * es)
        descs = [([p + lo * es for p in dins], [p + lo * es for p in douts], hi - lo)
                 for lo, hi in zip(edges[:-1], edges[1:]) if (lo // 7) % 5]            # leave some gaps untouched
        N.check(K.reduce_bcast_slices(descs, k, nout, dtype, N.OP_SUM), "fx_reduce_bcast_slices")
        dev.sync()
        expect = np.frombuffer(bytes([0x5A]) * (total * es), dtype=npdt).copy()
        for lo, hi in zip(edges[:-1], edges[1:]):
            if (lo // 7) % 5:
                expect[lo:hi] = want[lo:hi]
        for d in douts:
            assert np.array_equal(dev.to_host(d, total, npdt).view(np.uint8), expect.view(np.uint8))
    # broadcast copy: one source, five destinations, byte granular
    src = np.random.default_rng(6).integers(0, 256, 100003, dtype=np.uint8)
    with DevBufs(dev) as b:
        dsrc = b.put(src, pad_before=3)
        dd = [b.alloc(src.size + 64) + 3 for _ in range(5)]
        N.check(K.reduce_bcast_slices([([dsrc], dd, src.size)], 1, 5, 0, -1), "broadcast copy")
        dev.sync()
        for d in dd:
            assert np.array_equal(dev.to_host(d, src.size, np.uint8), src)


def test_more_slices_than_one_kernel_argument_table_holds(dev):
    """500 disjoint, non-adjacent copies (the table for copies holds 142) and 300
    two-input reduces (110 per table) in one call each: several launches, every
    slice executed exactly once, gaps untouched."""
    rng = np.random.default_rng(9)
    nsl, seg, gap = 500, 777, 13
    src = rng.integers(0, 256, nsl * (seg + gap), dtype=np.uint8)
    with DevBufs(dev) as b:
        dsrc, ddst = b.put(src), b.alloc(src.size)
        dev.memset(ddst, 0xEE, src.size)
        N.check(K.copy_slices([(dsrc + i * (seg + gap), ddst + i * (seg + gap), seg) for i in range(nsl)]))
        dev.sync()
        got = dev.to_host(ddst, src.size, np.uint8).reshape(nsl, seg + gap)
    want = src.reshape(nsl, seg + gap).copy()
    want[:, seg:] = 0xEE
    assert np.array_equal(got, want)
    nsl, seg, gap = 300, 1001, 3
    a, c = seeded_inputs(N.DT_FP32, 2, nsl * (seg + gap), seed=17)
    full = O.reduce2(a, c, N.DT_FP32, N.OP_SUM)
    with DevBufs(dev) as b:
        da, dc, do = b.put(a), b.put(c), b.alloc(a.nbytes)
        dev.memset(do, 0, a.nbytes)
        descs = [([da + 4 * i * (seg + gap), dc + 4 * i * (seg + gap)], do + 4 * i * (seg + gap), seg) for i in range(nsl)]
        N.check(K.reduce_slices(descs, 2, N.DT_FP32, N.OP_SUM))
        dev.sync()
        got = dev.to_host(do, a.size, np.float32).reshape(nsl, seg + gap)
    want = full.reshape(nsl, seg + gap).copy()
    want[:, seg:] = 0
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("dname", ["bf16", "fp16"])
def test_element_fold_is_the_reference_device_kernels_arithmetic(dev, dname):
    """op | FX_OP_ELEMENT_FOLD: the 16-bit types folded in the element type, as
    lsa_reduce does (custom_allreduce.cu:326-361) -- rounded after every
    addition, max / min handing on the later operand on ties and NaN.  Bit for
    bit against the oracle's restatement (NaN for NaN where a sum makes one),
    through the direct kernel, the slice table, the multi-output kernel and the
    run-time-k kernels; specials sprinkled over random data."""
    dtype = DTYPES[dname]
    ELEM = 0x100
    rng = np.random.default_rng(11)
    specials = np.array([0x0000, 0x8000, 0x7FC0 if dname == "bf16" else 0x7E00, 0x7F80 if dname == "bf16" else 0x7C00,
                         0xFF80 if dname == "bf16" else 0xFC00, 0x0001, 0x8001, 0x4380, 0x3F80, 0x6800, 0x3C00], np.uint16)

    def inputs(k, n, seed):
        ins = seeded_inputs(dtype, k, n, seed=seed, dist=(0.0, 300.0))      # large enough that step rounding shows
        for a in ins:
            where = rng.random(n) < 0.02
            a[where] = rng.choice(specials, int(where.sum()))
        return ins

    def same(got, want, op, what):
        if op == N.OP_SUM:
            gn, wn = is_nan16(got, dtype), is_nan16(want, dtype)
            assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
            assert np.array_equal(got[~gn], want[~wn]), what
        else:
            assert np.array_equal(got, want), what

    differs = 0
    for op in (N.OP_SUM, N.OP_MAX, N.OP_MIN):
        for k, n, first, mis in [(1, 1001, 0, 0), (2, 40001, 1, 1), (3, 7, 2, 0), (5, 300007, 0, 3), (8, 1 << 20, 5, 0),
                                 (12, 70001, 7, 1), (33, 4099, 0, 0)]:
            ins = inputs(k, n, seed=k * 10 + op)
            want = O.reduce_copy_elem(ins, dtype, op, first=first)
            differs += int((want != O.reduce_copy(ins, dtype, op, first=first)).sum())
            with DevBufs(dev) as b:
                dins = [b.put(a, pad_before=mis * 2) for a in ins]
                out = b.alloc(n * 2 + 64)
                N.check(K.reduce_copy(out, dins, n, dtype, op | ELEM, first), f"fx_reduce_copy k={k}")
                dev.sync()
                same(dev.to_host(out, n, np.uint16), want, op, f"{dname} op={op} k={k} n={n} direct")
                if k <= 8:                                   # the slice table and the multi-output kernel, in two pieces
                    rot = [dins[(first + j) % k] for j in range(k)]
                    cut = n // 3
                    outs = [b.alloc(n * 2 + 64) for _ in range(3)]
                    descs = [(rot, outs[0], cut), ([p + cut * 2 for p in rot], outs[0] + cut * 2, n - cut)]
                    N.check(K.reduce_slices(descs, k, dtype, op | ELEM), "fx_reduce_slices")
                    bd = [(rot, outs[1:], cut), ([p + cut * 2 for p in rot], [o + cut * 2 for o in outs[1:]], n - cut)]
                    N.check(K.reduce_bcast_slices(bd, k, 2, dtype, op | ELEM), "fx_reduce_bcast_slices")
                    dev.sync()
                    for o in outs:
                        same(dev.to_host(o, n, np.uint16), want, op, f"{dname} op={op} k={k} slices / bcast")
                else:
                    outs = [b.alloc(n * 2 + 64) for _ in range(k)]
                    N.check(K.reduce_bcast(outs, dins, n, dtype, op | ELEM, first), "fx_reduce_bcast")
                    dev.sync()
                    for o in outs[:: max(k // 3, 1)]:
                        same(dev.to_host(o, n, np.uint16), want, op, f"{dname} op={op} k={k} run-time k")
    assert differs > 1000, "the inputs never showed the difference from the default arithmetic"
    # what the reference kernel's dispatch refuses (custom_allreduce.cu:498-518)
    assert K.reduce_copy(16, [16, 32], 4, dtype, N.OP_PROD | ELEM) == N.NOT_SUPPORTED
    assert K.reduce_copy(16, [16, 32], 4, dtype, N.OP_AVG | ELEM) == N.NOT_SUPPORTED
    assert K.reduce_copy(16, [16, 32], 4, N.DT_FP32, N.OP_MAX | ELEM) == N.NOT_SUPPORTED
    assert K.reduce_copy(16, [16, 32], 4, N.DT_INT32, N.OP_SUM | ELEM) == N.NOT_SUPPORTED
    assert K.reduce_copy(16, [16, 32], 4, dtype, 7 | ELEM) == N.INVALID_ARGUMENT


@pytest.mark.parametrize("n,block,smis,rmis", [(1, 7, 0, 0), (2, 1, 1, 3), (3, 4099, 2, 0), (8, 64 << 10, 0, 0), (8, (1 << 20) + 36, 4, 4),
                                               (13, 30001, 0, 1), (33, 1000, 0, 0), (64, 516, 4, 8), (5, 3 << 20, 0, 0)])
def test_alltoall_in_one_launch(dev, n, block, smis, rmis):
    """fx_alltoall: block i of send[r] becomes block r of recv[i] for every
    pair, whatever the alignment of the buffers and the block size (odd sizes,
    blocks long enough for the striped hand-out, 64 ranks); nothing is written
    outside the n * block bytes of a receive buffer."""
    rng = np.random.default_rng(n * 7 + block)
    sends = [rng.integers(0, 256, n * block, dtype=np.uint8) for _ in range(n)]
    with DevBufs(dev) as b:
        ds = [b.put(a, pad_before=smis) for a in sends]
        dr = []
        for r in range(n):
            base = b.alloc(16 + rmis + n * block + 64)
            dev.memset(base, 0xA5, 16 + rmis + n * block + 64)
            dr.append(base + 16 + rmis)
        dev.sync()
        N.check(K.alltoall(dr, ds, block), "fx_alltoall")
        dev.sync()
        for i in range(n):
            got = dev.to_host(dr[i] - 16, 16 + n * block + 32, np.uint8)
            want = np.concatenate([sends[r][i * block:(i + 1) * block] for r in range(n)])
            assert (got[:16] == 0xA5).all() and (got[16 + n * block:] == 0xA5).all(), f"rank {i}: wrote outside its buffer"
            assert np.array_equal(got[16:16 + n * block], want), f"rank {i}"
    assert K.alltoall([16] * 65, [16] * 65, 4) == N.INVALID_ARGUMENT
    assert K.alltoall([16, 0], [16, 32], 4) == N.INVALID_ARGUMENT
    assert K.alltoall([16], [32], 0) == N.SUCCESS
