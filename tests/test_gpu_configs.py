"""The five configurations of BASELINE.json at their FULL sizes on the GPU: bit-exact
against committed digests of the oracle's output, against the oracle run live on
this box's host cores, and through size-independent properties."""
import json
import os

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from flagcx_amd import sim as S
from oracle import fx_oracle as O
from tests.golden import workloads as W
from tests.util import DevBufs, assert_parity

pytestmark = pytest.mark.gpu
GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "golden.json")))
THREADS = min(16, len(os.sched_getaffinity(0)))


@pytest.fixture(scope="module", autouse=True)
def _threads():
    O.lib.oracle_set_threads(THREADS)
    yield
    O.lib.oracle_set_threads(1)


@pytest.fixture()
def stream(dev):
    s = dev.stream_create()
    yield s
    dev.stream_destroy(s)


def test_cfg1_fp32_sum_two_inputs(dev):
    c = W.CFG1
    ins = W.inputs(c["dtype"], c["k"], c["n"], c["dist"], c["seed"], THREADS)
    with DevBufs(dev) as b:
        dins = [b.put(a) for a in ins]
        dout = b.alloc(c["n"] * 4)
        N.check(K.reduce_copy(dout, dins, c["n"], c["dtype"], N.OP_SUM))
        dev.sync()
        got = dev.to_host(dout, c["n"], np.float32)
    assert W.digest(got) == GOLDEN["cfg1_fp32_sum_2x16777216"]["out_sha256"]
    assert_parity(got, O.reduce2(ins[0], ins[1], c["dtype"], N.OP_SUM), c["dtype"], N.OP_SUM, "cfg1")


def test_cfg2_ring_share_slices_then_allgather(dev, stream):
    """8 simulated peers x 33,554,432 bf16: every rank's reduce-scatter share cut
    into 8 slices and 512 KiB (262,144-element) pieces -- 128 descriptors, 8-way,
    fp32 accumulate -- then the all-gather copy phase; plus the whole thing through
    flagcxAllReduce."""
    c = W.CFG2
    n, k = c["n"], c["k"]
    want_digest = GOLDEN["cfg2_bf16_sum_8x33554432"]["out_sha256"]
    ins = W.inputs(c["dtype"], k, n, c["dist"], c["seed"], THREADS)
    assert [W.digest(a) for a in ins] == GOLDEN["cfg2_bf16_sum_8x33554432"]["inputs_sha256"]
    nred = N.lib.fx_nredslices(n, k, c["nslices"], 0, c["redslice_elems"])
    assert nred == 2
    with DevBufs(dev) as b:
        ds = [b.put(a) for a in ins]
        dr = [b.alloc(n * 2) for _ in range(k)]
        # (i) rank shares as explicit descriptors: chunk -> slice -> red-slice, owner = (chunk-1) % k
        descs, copies = [], []
        for ch in range(k):
            ccnt, coff = K.split(n, k, ch)
            owner = (ch - 1) % k
            for s in range(c["nslices"]):
                scnt, soff = K.split(ccnt, c["nslices"], s)
                for q in range(nred):
                    rcnt, roff = K.split(scnt, nred, q)
                    assert rcnt == c["redslice_elems"]
                    off = (coff + soff + roff) * 2
                    descs.append(([p + off for p in ds], dr[owner] + off, rcnt))
            copies += [(dr[owner] + coff * 2, dr[r] + coff * 2, ccnt * 2) for r in range(k) if r != owner]
        assert len(descs) == 128
        raw = dev.raw_stream(stream)
        N.check(K.reduce_slices(descs, k, c["dtype"], N.OP_SUM, raw))
        N.check(K.copy_slices(copies, raw))
        dev.stream_sync(stream)
        for r in (0, 3, 7):
            assert W.digest(dev.to_host(dr[r], n, np.uint16)) == want_digest, f"rank {r}"
        # (ii) the same through the collective entry point
        for p in dr:
            dev.memset(p, 0, n * 2)
        with S.SimGroup(k, nslices=c["nslices"], redslicesize=c["redslice_elems"]) as g:
            N.check(g.all_reduce(ds, dr, n, c["dtype"], N.OP_SUM, stream))
            dev.stream_sync(stream)
        got = dev.to_host(dr[5], n, np.uint16)
        assert W.digest(got) == want_digest
        # live oracle on one share
        ccnt, coff = K.split(n, k, 2)
        assert_parity(got[coff:coff + ccnt], O.reduce_copy([a[coff:coff + ccnt] for a in ins], c["dtype"], N.OP_SUM),
                      c["dtype"], N.OP_SUM, "cfg2 share 2")


@pytest.mark.parametrize("dtype", list(W.CFG3["dists"]))
def test_cfg3_size_and_op_sweep(dev, dtype):
    """k = 4, 1 KiB .. 1 GiB per input at every power of two, sum/max/min/prod, in
    place and out of place.  Up to 16 MiB every case is compared with the
    committed digests; above, with the oracle run live on the same inputs."""
    es = N.DTYPE_SIZE[dtype]
    nmax = (1 << 30) // es
    ins = W.cfg3_inputs(dtype, nmax, THREADS)
    name = W.DTYPE_NAMES[dtype]
    with DevBufs(dev) as b:
        dins = [b.put(a) for a in ins]
        dout = b.alloc(nmax * es)
        dscratch = b.alloc(nmax * es)                     # in-place runs work on a copy of input 0
        for lg in range(10, 31):
            n = (1 << lg) // es
            for oname, op in W.OPS.items():
                if lg <= 24:
                    want_digest, want = GOLDEN["cfg3"][f"{name}_{oname}_{1 << lg}"]["out_sha256"], None
                else:
                    want_digest, want = None, O.reduce_copy([a[:n] for a in ins], dtype, op)
                N.check(K.reduce_copy(dout, dins, n, dtype, op))
                dev.copy(dscratch, dins[0], n * es)
                N.check(K.reduce_copy(dscratch, [dscratch] + dins[1:], n, dtype, op))     # out = in[0]
                dev.sync()
                for label, ptr in (("out-of-place", dout), ("in-place", dscratch)):
                    got = dev.to_host(ptr, n, N.NP_DTYPE[dtype])
                    same = (W.digest(got) == want_digest) if want is None else \
                        np.array_equal(got.view(np.uint8), want.view(np.uint8))
                    if not same:                          # fp16 sum/prod may differ by 1 ulp at most: show it
                        want = want if want is not None else O.reduce_copy([a[:n] for a in ins], dtype, op)
                        assert_parity(got, want, dtype, op, f"cfg3 {name} {oname} {1 << lg} B {label}")
                        if dtype != N.DT_FP16 or op in (N.OP_MAX, N.OP_MIN):
                            raise AssertionError(f"cfg3 {name} {oname} {1 << lg} B {label}: digest differs")


def test_cfg4_alltoallv_pack_unpack(dev):
    e = GOLDEN["cfg4_alltoallv_pack_unpack"]
    counts, sd, slen, rd, rlen = W.cfg4_layout()
    assert counts == e["counts"] and sd == e["sdispls"] and rd == e["rdispls"]
    send = W.inputs(N.DT_FP32, 1, slen, (0, -1.0, 1.0), W.CFG4["seed"], THREADS)[0]
    total = sum(counts)
    with DevBufs(dev) as b:
        dsend, dpacked, drecv = b.put(send), b.alloc(total * 4), b.alloc(rlen * 4)
        dev.memset(drecv, 0, rlen * 4)
        N.check(K.pack(dpacked, dsend, counts, sd, N.DT_FP32))
        N.check(K.unpack(drecv, dpacked, counts, rd, N.DT_FP32))
        dev.sync()
        packed = dev.to_host(dpacked, total, np.float32)
        recv = dev.to_host(drecv, rlen, np.float32)
        # scatter back to the ORIGINAL displacements restores the touched ranges of the send buffer
        dback = b.alloc(slen * 4)
        dev.memset(dback, 0, slen * 4)
        N.check(K.unpack(dback, dpacked, counts, sd, N.DT_FP32))
        dev.sync()
        back = dev.to_host(dback, slen, np.float32)
    assert W.digest(packed) == e["packed_sha256"]
    assert W.digest(recv) == e["unpacked_sha256"]
    touched = np.zeros(slen, bool)
    for c_, d_ in zip(counts, sd):
        touched[d_:d_ + c_] = True
    assert np.array_equal(back[touched].view(np.uint32), send[touched].view(np.uint32))
    assert (back[~touched].view(np.uint32) == 0).all()


def test_cfg5_large_bf16_sum(dev, stream):
    """8 x 268,435,456 bf16 (512 MiB each): one launch out of place, in place,
    and streamed as 128 chunks of 4 MiB; all three must hash to the committed
    digest of the oracle's output.  Then properties that need no oracle."""
    c = W.CFG5
    n, k = c["n"], c["k"]
    gold = GOLDEN["cfg5_bf16_sum_8x268435456"]
    raw = dev.raw_stream(stream)
    with DevBufs(dev) as b:
        dins = []
        for p in range(k):
            host = K.synth(n, c["dtype"], *c["dist"], c["seed"], p, THREADS)
            assert W.digest(host) == gold["inputs_sha256"][p], f"input {p}"
            dins.append(b.put(host))
            if p == 0:
                first = host
        del host
        dout = b.alloc(n * 2)
        N.check(K.reduce_copy(dout, dins, n, c["dtype"], N.OP_SUM, 0, raw))
        dev.stream_sync(stream)
        got = dev.to_host(dout, n, np.uint16)
        assert W.probe(got) == gold["out_probe"]
        assert W.digest(got) == gold["out_sha256"], "out-of-place"
        # streamed in 4 MiB chunks: 128 descriptors
        dev.memset(dout, 0, n * 2)
        chunk = (4 << 20) // 2
        descs = [([p + i * chunk * 2 for p in dins], dout + i * chunk * 2, chunk) for i in range(n // chunk)]
        assert len(descs) == 128
        N.check(K.reduce_slices(descs, k, c["dtype"], N.OP_SUM, raw))
        dev.stream_sync(stream)
        assert W.digest(dev.to_host(dout, n, np.uint16)) == gold["out_sha256"], "4 MiB chunks"
        # properties: max over identical inputs is the identity; x + 0 + ... + 0 == x up to the sign of zero
        N.check(K.reduce_copy(dout, [dins[0]] * k, n, c["dtype"], N.OP_MAX, 0, raw))
        dev.stream_sync(stream)
        assert np.array_equal(dev.to_host(dout, n, np.uint16), first)
        dzero = b.alloc(n * 2)
        dev.memset(dzero, 0, n * 2)
        N.check(K.reduce_copy(dout, [dins[0]] + [dzero] * (k - 1), n, c["dtype"], N.OP_SUM, 0, raw))
        dev.stream_sync(stream)
        ident = dev.to_host(dout, n, np.uint16)
        assert np.array_equal(np.where(ident == 0x8000, 0, ident), np.where(first == 0x8000, 0, first))
        # in place (out = in[0]); last, because it overwrites input 0
        N.check(K.reduce_copy(dins[0], dins, n, c["dtype"], N.OP_SUM, 0, raw))
        dev.stream_sync(stream)
        assert W.digest(dev.to_host(dins[0], n, np.uint16)) == gold["out_sha256"], "in-place"


@pytest.mark.parametrize("dname,dtype,count", [("int8", N.DT_INT8, (1 << 32) + (3 << 20) + 12345),   # > 2^32 elements
                                               ("fp32", N.DT_FP32, (1 << 31) + 777)])             # > 2^33 bytes
def test_counts_beyond_32_bit_offsets(dev, dname, dtype, count):
    """Maximum sizes: element counts and byte offsets that do not fit 32 bits.
    Inputs are a byte pattern with seeded random patches planted at the start,
    across the 2^32-byte boundary and at the end, so that an index truncated to
    32 bits would read the wrong patch.  The whole output is downloaded and
    compared piecewise with the oracle; the bytes behind it must be untouched."""
    es = N.DTYPE_SIZE[dtype]
    npdt = N.NP_DTYPE[dtype]
    nbytes = count * es
    patch_el = (1 << 20) // es
    starts = sorted({0, ((1 << 32) - (1 << 19)) // es, count - patch_el})          # element offsets of the patches
    assert all(s + patch_el <= count for s in starts)
    rng = np.random.default_rng(count % 1000)
    fill = (0x01, 0x02)
    with DevBufs(dev) as b:
        dins, patches = [], []
        for p in range(2):
            d = b.alloc(nbytes + 256)
            dev.memset(d, fill[p], nbytes)
            mine = {}
            for s in starts:
                raw = rng.integers(0, 256, patch_el * es, dtype=np.uint8)
                if dtype == N.DT_FP32:                                                # finite values only
                    with np.errstate(all="ignore"):
                        f = raw.view(np.float32) % np.float32(1e6)
                    raw = np.nan_to_num(f, nan=1.5).view(np.uint8)
                mine[s] = raw.view(npdt)
                dev.upload(d + s * es, mine[s])
            dins.append(d)
            patches.append(mine)
        dout = b.alloc(nbytes + 256)
        dev.memset(dout, 0xEE, nbytes + 256)
        N.check(K.reduce_copy(dout, dins, count, dtype, N.OP_SUM), "fx_reduce_copy")
        dev.sync()
        base = [np.full(1, f, np.uint8).repeat(es).view(npdt)[0] for f in fill]
        plain = O.reduce2(np.full(4, base[0], npdt), np.full(4, base[1], npdt), dtype, N.OP_SUM)[0]
        step = (1 << 28) // es                                                        # 256 MiB per download
        for off in range(0, count, step):
            n = min(step, count - off)
            got = dev.to_host(dout + off * es, n, npdt)
            want = np.full(n, plain, npdt)
            for s in starts:
                lo, hi = max(s, off), min(s + patch_el, off + n)
                if lo < hi:
                    a = [np.full(hi - lo, base[p], npdt) for p in range(2)]
                    for p in range(2):
                        a[p][:] = patches[p][s][lo - s:hi - s]
                    want[lo - off:hi - off] = O.reduce2(a[0], a[1], dtype, N.OP_SUM)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), f"{dname}: window at element {off}"
        assert (dev.to_host(dout + nbytes, 256, np.uint8) == 0xEE).all(), "wrote past the end"


def test_cfg5_through_the_collective(dev, stream):
    """The headline workload as one flagcxAllReduce over 8 simulated ranks (every
    rank sends 512 MiB of bf16, every rank receives the 8-way sum): first and
    last rank's results hash to the committed digest, the others agree with them
    on sampled windows."""
    c = W.CFG5
    n, k = c["n"], c["k"]
    gold = GOLDEN["cfg5_bf16_sum_8x268435456"]
    with DevBufs(dev) as b, S.SimGroup(k) as g:
        ds = []
        for p in range(k):
            host = K.synth(n, c["dtype"], *c["dist"], c["seed"], p, THREADS)
            ds.append(b.put(host))
        del host
        dr = [b.alloc(n * 2) for _ in range(k)]
        N.check(g.all_reduce(ds, dr, n, c["dtype"], N.OP_SUM, stream), "flagcxAllReduce")
        dev.stream_sync(stream)
        first = dev.to_host(dr[0], n, np.uint16)
        assert W.digest(first) == gold["out_sha256"], "rank 0"
        assert W.digest(dev.to_host(dr[k - 1], n, np.uint16)) == gold["out_sha256"], f"rank {k - 1}"
        win = 1 << 19
        for r in range(1, k - 1):
            for pos in np.linspace(0, n - win, 9).astype(np.int64):
                got = dev.to_host(dr[r] + int(pos) * 2, win, np.uint16)
                assert np.array_equal(got, first[pos:pos + win]), f"rank {r} window at {pos}"


def test_half_the_hbm_in_one_launch(dev):
    """Sized for the part: 8 inputs of 16 GiB (2^33 + 12,345 bf16 elements each) and
    a 16 GiB output -- 144 GiB resident, 524,289 workgroups, element counts and byte
    offsets far beyond 32 bits -- in ONE fx_reduce_copy.  Inputs are byte patterns
    with seeded random patches at the start, across every 4 GiB boundary and at
    the ragged end; the whole output is downloaded window by window and compared
    with the oracle, and the bytes behind it must be untouched."""
    k, dtype, es = 8, N.DT_BF16, 2
    count = (1 << 33) + 12345
    nbytes = count * es
    patch_el = 1 << 19                                                   # 1 MiB of bf16
    starts = sorted({0, count - patch_el} | {(g << 32) // es - patch_el // 2 for g in range(1, 4)})
    rng = np.random.default_rng(8)
    fills = [0x3c + p for p in range(k)]                                  # bf16 0x3c3c .. 0x4343: finite, distinct
    with DevBufs(dev) as b:
        try:
            dins = [b.alloc(nbytes + 256) for _ in range(k)]
            dout = b.alloc(nbytes + 256)
        except RuntimeError as e:                                        # a smaller part, or memory in use
            pytest.skip(f"cannot hold 144 GiB on this device: {e}")
        patches = []
        for p in range(k):
            dev.memset(dins[p], fills[p], nbytes)
            mine = {}
            for s in starts:
                bits = rng.integers(0, 1 << 16, patch_el, dtype=np.uint16)
                bits[(bits & 0x7f80) == 0x7f80] = 0x3f80                 # no inf / NaN: keep the sum's bits defined
                mine[s] = bits
                dev.upload(dins[p] + s * es, bits)
            patches.append(mine)
        dev.memset(dout, 0xEE, nbytes + 256)
        N.check(K.reduce_copy(dout, dins, count, dtype, N.OP_SUM), "fx_reduce_copy")
        dev.sync()
        base = [np.uint16(f << 8 | f) for f in fills]
        plain = O.reduce_copy([np.full(4, v, np.uint16) for v in base], dtype, N.OP_SUM)[0]
        step = 1 << 27                                                   # 256 MiB of bf16 per download
        for off in range(0, count, step):
            n = min(step, count - off)
            got = dev.to_host(dout + off * es, n, np.uint16)
            want = np.full(n, plain, np.uint16)
            for s in starts:
                lo, hi = max(s, off), min(s + patch_el, off + n)
                if lo < hi:
                    want[lo - off:hi - off] = O.reduce_copy([patches[p][s][lo - s:hi - s] for p in range(k)], dtype, N.OP_SUM)
            assert np.array_equal(got, want), f"window at element {off}"
        assert (dev.to_host(dout + nbytes, 256, np.uint8) == 0xEE).all(), "wrote past the end"
