"""torch.distributed collectives through the "flagcx" backend (flagcx_amd/
torch_backend), run as a process of its own by tests/test_gpu_torch.py with
torch imported first.  n simulated ranks, one backend object each, share a
HashStore; every rank posts, then every Work is waited for, and the tensors are
compared bit for bit with the CPU oracle (reductions) or with the inputs (data
movement).  A one-rank group goes through torch.distributed.init_process_group
and the module-level API.  Prints "torch backend ok" at the end."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import torch                                    # noqa: E402  (first on purpose)
import numpy as np
import torch.distributed as dist
from torch.distributed import ReduceOp

import flagcx_amd.torch_backend as fxb
from flagcx_amd import _native as N
from flagcx_amd import comm
from oracle import fx_oracle as O

BITS = {torch.bfloat16: torch.int16, torch.float16: torch.int16, torch.float32: torch.int32, torch.int32: torch.int32,
        torch.int64: torch.int64, torch.float64: torch.int64, torch.uint8: torch.uint8, torch.int8: torch.int8}


def words(t):
    dt = comm.dtype_code(t.dtype)
    return t.detach().contiguous().view(BITS[t.dtype]).cpu().numpy().view(N.NP_DTYPE[dt])


def make(dtype, shape, gen):
    if dtype.is_floating_point:
        return (torch.randn(shape, device="cuda", generator=gen, dtype=torch.float32) * 3).to(dtype)
    info = torch.iinfo(dtype)
    return torch.randint(max(info.min, -1000), min(info.max, 1000), shape, device="cuda", generator=gen, dtype=dtype)


def same(got, want, what):
    g, w = np.ascontiguousarray(got).view(np.uint8).ravel(), np.ascontiguousarray(want).view(np.uint8).ravel()
    if g.shape != w.shape or not np.array_equal(g, w):
        bad = np.flatnonzero(g != w) if g.shape == w.shape else []
        raise SystemExit(f"{what}: results differ ({len(bad)} of {g.size} bytes, first at {bad[0] if len(bad) else -1}; shapes {g.shape} {w.shape})")


def wait_all(works):
    for w in works:
        assert w.wait()
    torch.cuda.synchronize()


def simulated(n, gen):
    store = dist.HashStore()
    ranks = [fxb.new_backend(store, r, n) for r in range(n)]
    assert [b.rank() for b in ranks] == list(range(n)) and all(b.size() == n for b in ranks)
    assert ranks[0].name() == "flagcx"

    # all-reduce: every dtype the backend maps, sum / max / avg / product
    for dtype, op in [(torch.bfloat16, ReduceOp.SUM), (torch.float16, ReduceOp.MAX), (torch.float32, ReduceOp.SUM),
                      (torch.float32, ReduceOp.AVG), (torch.float64, ReduceOp.PRODUCT), (torch.int32, ReduceOp.MIN),
                      (torch.int64, ReduceOp.SUM), (torch.uint8, ReduceOp.MAX), (torch.int8, ReduceOp.SUM)]:
        ts = [make(dtype, (257, 1031), gen) for _ in range(n)]
        want = O.reduce_copy([words(t) for t in ts], comm.dtype_code(dtype), comm.op_code(op))
        opts = dist.AllreduceOptions()
        opts.reduceOp = op
        wait_all([b.allreduce([t], opts) for b, t in zip(ranks, ts)])
        for r, t in enumerate(ts):
            same(words(t).ravel(), want, f"allreduce {dtype} {op} rank {r}")
        print(f"ok  allreduce {dtype} {op}", flush=True)

    # booleans: a sum is an "or"
    bs = [torch.rand(5000, device="cuda", generator=gen) < 0.2 for _ in range(n)]
    want = torch.stack(bs).any(0)
    wait_all([b.allreduce([t]) for b, t in zip(ranks, bs)])
    assert all(torch.equal(t, want) for t in bs)
    print("ok  allreduce bool", flush=True)

    # a side stream: the collective is ordered after the producer on that stream, the consumer after wait()
    side = torch.cuda.Stream()
    ts = [torch.zeros(1 << 20, device="cuda") for _ in range(n)]
    with torch.cuda.stream(side):
        for r, t in enumerate(ts):
            t.add_(float(r + 1))
        works = [b.allreduce([t]) for b, t in zip(ranks, ts)]
    for w in works:
        w.wait()                                  # orders the default stream after the side stream's work
    total = sum(t.sum() for t in ts)
    assert float(total) == n * (n * (n + 1) / 2) * (1 << 20), float(total)
    print("ok  allreduce on a side stream", flush=True)

    # broadcast / reduce
    ts = [make(torch.float32, (3, 70001), gen) for _ in range(n)]
    src = ts[2].clone()
    o = dist.BroadcastOptions()
    o.rootRank = 2
    wait_all([b.broadcast([t], o) for b, t in zip(ranks, ts)])
    assert all(torch.equal(t, src) for t in ts)
    ts = [make(torch.bfloat16, (99991,), gen) for _ in range(n)]
    want = O.reduce_copy([words(t) for t in ts], N.DT_BF16, N.OP_SUM)
    keep = [t.clone() for t in ts]
    o = dist.ReduceOptions()
    o.rootRank = 1
    wait_all([b.reduce([t], o) for b, t in zip(ranks, ts)])
    same(words(ts[1]), want, "reduce root")
    assert all(torch.equal(ts[r], keep[r]) for r in range(n) if r != 1), "reduce touched a non-root tensor"
    print("ok  broadcast, reduce", flush=True)

    # all-gather: into one tensor, and into a list of tensors
    ins = [make(torch.float16, (4099,), gen) for _ in range(n)]
    outs = [torch.empty(n * 4099, device="cuda", dtype=torch.float16) for _ in range(n)]
    wait_all([b._allgather_base(o_, i_) for b, o_, i_ in zip(ranks, outs, ins)])
    assert all(torch.equal(o_, torch.cat(ins)) for o_ in outs)
    lists = [[torch.empty(17, 241, device="cuda", dtype=torch.int32) for _ in range(n)] for _ in range(n)]
    ins = [make(torch.int32, (17, 241), gen) for _ in range(n)]
    wait_all([b.allgather([l], [i_]) for b, l, i_ in zip(ranks, lists, ins)])
    assert all(torch.equal(lists[r][q], ins[q]) for r in range(n) for q in range(n))
    print("ok  all-gather (tensor, list)", flush=True)

    # reduce-scatter: from one tensor, and from a list
    ins = [make(torch.float32, (n * 30011,), gen) for _ in range(n)]
    outs = [torch.empty(30011, device="cuda") for _ in range(n)]
    want = O.reduce_copy([words(t) for t in ins], N.DT_FP32, N.OP_SUM)
    wait_all([b._reduce_scatter_base(o_, i_) for b, o_, i_ in zip(ranks, outs, ins)])
    for r in range(n):
        same(words(outs[r]), want[r * 30011:(r + 1) * 30011], f"reduce_scatter_tensor rank {r}")
    lists = [[make(torch.bfloat16, (5, 1001), gen) for _ in range(n)] for _ in range(n)]
    outs = [torch.empty(5, 1001, device="cuda", dtype=torch.bfloat16) for _ in range(n)]
    wait_all([b.reduce_scatter([o_], [l]) for b, o_, l in zip(ranks, outs, lists)])
    for r in range(n):
        want = O.reduce_copy([words(lists[q][r]).ravel() for q in range(n)], N.DT_BF16, N.OP_SUM)
        same(words(outs[r]).ravel(), want, f"reduce_scatter list rank {r}")
    print("ok  reduce-scatter (tensor, list)", flush=True)

    # all-to-all: equal pieces, row splits, lists of tensors
    ins = [make(torch.int64, (n * 1000,), gen) for _ in range(n)]
    outs = [torch.empty_like(t) for t in ins]
    wait_all([b.alltoall_base(o_, i_, [], []) for b, o_, i_ in zip(ranks, outs, ins)])
    for r in range(n):
        assert torch.equal(outs[r], torch.cat([ins[q][r * 1000:(r + 1) * 1000] for q in range(n)]))
    split = [[(r + q) % 3 + (q == 1) for q in range(n)] for r in range(n)]        # rank r sends split[r][q] rows to q
    ins = [make(torch.float32, (sum(split[r]), 7), gen) for r in range(n)]
    outs = [torch.empty(sum(split[q][r] for q in range(n)), 7, device="cuda") for r in range(n)]
    wait_all([b.alltoall_base(outs[r], ins[r], [split[q][r] for q in range(n)], split[r]) for r, b in enumerate(ranks)])
    for r in range(n):
        parts = []
        for q in range(n):
            lo = sum(split[q][:r])
            parts.append(ins[q][lo:lo + split[q][r]])
        assert torch.equal(outs[r], torch.cat(parts)), f"all_to_all_single with splits, rank {r}"
    il = [[make(torch.float16, (3 + r + q,), gen) for q in range(n)] for r in range(n)]
    ol = [[torch.empty(3 + q + r, device="cuda", dtype=torch.float16) for q in range(n)] for r in range(n)]
    wait_all([b.alltoall(ol[r], il[r]) for r, b in enumerate(ranks)])
    assert all(torch.equal(ol[r][q], il[q][r]) for r in range(n) for q in range(n))
    print("ok  all-to-all (equal, splits, lists)", flush=True)

    # gather / scatter / send / recv / barrier
    ins = [make(torch.float32, (1234,), gen) for _ in range(n)]
    got = [torch.empty(1234, device="cuda") for _ in range(n)]
    o = dist.GatherOptions()
    o.rootRank = 3
    wait_all([b.gather([got] if r == 3 else [], [ins[r]], o) for r, b in enumerate(ranks)])
    assert all(torch.equal(got[q], ins[q]) for q in range(n))
    outs = [torch.empty(777, device="cuda", dtype=torch.int32) for _ in range(n)]
    parts = [make(torch.int32, (777,), gen) for _ in range(n)]
    o = dist.ScatterOptions()
    o.rootRank = 0
    wait_all([b.scatter([outs[r]], [parts] if r == 0 else [], o) for r, b in enumerate(ranks)])
    assert all(torch.equal(outs[r], parts[r]) for r in range(n))
    msg, box = make(torch.bfloat16, (65537,), gen), torch.empty(65537, device="cuda", dtype=torch.bfloat16)
    wait_all([ranks[1].send([msg], 2, 0), ranks[2].recv([box], 1, 0)])
    assert torch.equal(msg, box)
    wait_all([b.barrier() for b in ranks])
    print("ok  gather, scatter, send / recv, barrier", flush=True)

    # a coalescing bracket per rank (what batch_isend_irecv opens): the ring exchange, every rank sends right, receives left
    msgs = [make(torch.float32, (4099,), gen) for _ in range(n)]
    boxes = [torch.empty(4099, device="cuda") for _ in range(n)]
    works = []
    for r, b in enumerate(ranks):
        b._start_coalescing()
        b.send([msgs[r]], (r + 1) % n, 0)
        b.recv([boxes[r]], (r - 1) % n, 0)
        works.append(b._end_coalescing())
    wait_all(works)
    assert all(torch.equal(boxes[r], msgs[(r - 1) % n]) for r in range(n))
    print("ok  send / recv inside coalescing brackets", flush=True)

    # coalesced forms: one collective over all the tensors of the call, so that rank after rank can post them
    shapes = [(1001,), (3, 333), (70001,), (16,)]
    tl = [[make(torch.float32, sh, gen) for sh in shapes] for _ in range(n)]
    want = [O.reduce_copy([words(tl[r][i]).ravel() for r in range(n)], N.DT_FP32, N.OP_SUM) for i in range(len(shapes))]
    wait_all([b.allreduce_coalesced(ts) for b, ts in zip(ranks, tl)])
    for r in range(n):
        for i in range(len(shapes)):
            same(words(tl[r][i]).ravel(), want[i], f"allreduce_coalesced rank {r} tensor {i}")
    ext = fxb.extension()
    il = [[make(torch.bfloat16, sh, gen) for sh in shapes] for _ in range(n)]
    ol = [[torch.empty((n,) + sh, device="cuda", dtype=torch.bfloat16) for sh in shapes] for _ in range(n)]
    wait_all([ext.allgather_into_tensor_coalesced(b, ol[r], il[r]) for r, b in enumerate(ranks)])
    for r in range(n):
        for i in range(len(shapes)):
            assert torch.equal(ol[r][i], torch.stack([il[q][i] for q in range(n)])), f"allgather coalesced rank {r} tensor {i}"
    il = [[make(torch.float32, (n,) + sh, gen) for sh in shapes] for _ in range(n)]
    ol = [[torch.empty(sh, device="cuda") for sh in shapes] for _ in range(n)]
    wait_all([ext.reduce_scatter_tensor_coalesced(b, ol[r], il[r], ReduceOp.SUM) for r, b in enumerate(ranks)])
    for i in range(len(shapes)):
        want = O.reduce_copy([words(il[q][i]).ravel() for q in range(n)], N.DT_FP32, N.OP_SUM)
        per = want.size // n
        for r in range(n):
            same(words(ol[r][i]).ravel(), want[r * per:(r + 1) * per], f"reduce_scatter coalesced rank {r} tensor {i}")
    print("ok  coalesced all-reduce, all-gather, reduce-scatter", flush=True)

    # a Work that is dropped without a wait still fills its output list, and an input dropped right after the call
    # is still read
    ins = [make(torch.int32, (4001,), gen) for _ in range(n)]
    keep = [t.clone() for t in ins]
    lists = [[torch.zeros(4001, device="cuda", dtype=torch.int32) for _ in range(n)] for _ in range(n)]
    for r, b in enumerate(ranks):
        b.allgather([lists[r]], [ins[r]])
    del ins
    junk = [torch.full((4001,), -7, device="cuda", dtype=torch.int32) for _ in range(4 * n)]    # would reuse freed blocks
    torch.cuda.synchronize()
    assert all(torch.equal(lists[r][q], keep[q]) for r in range(n) for q in range(n)), "dropped Work / dropped input"
    del junk
    print("ok  dropped Work, dropped input", flush=True)

    # what the backend refuses
    o = dist.AllreduceOptions()
    o.reduceOp = ReduceOp.BAND
    t = torch.ones(8, device="cuda", dtype=torch.int32)
    for bad, kind in ((lambda: ranks[0].allreduce([t], o), ValueError),
                      (lambda: ranks[0].allreduce([t.cpu()]), RuntimeError),
                      (lambda: ranks[0].allreduce([torch.ones(4, 4, device="cuda").t()]), RuntimeError),
                      (lambda: ranks[0].allreduce([torch.ones(4, device="cuda", dtype=torch.complex64)]), TypeError)):
        try:
            bad()
        except kind:
            pass
        else:
            raise SystemExit("a call that should have been refused went through")
    print("ok  refusals", flush=True)
    del ranks


def two_groups_over_one_store(gen):
    """A second group built over the store of a first one must not pick up the
    first one's unique id -- not even when its rank 1 is built before its rank 0."""
    import threading
    import time
    store = dist.HashStore()
    first = [fxb.new_backend(store, r, 2) for r in range(2)]
    box = {}
    th = threading.Thread(target=lambda: box.__setitem__(1, fxb.new_backend(store, 1, 2)))
    th.start()
    time.sleep(0.3)                      # rank 1 of the second group is now waiting for ITS rank 0
    assert 1 not in box, "rank 1 of the second group did not wait for its own rank 0"
    box[0] = fxb.new_backend(store, 0, 2)
    th.join(30)
    assert not th.is_alive() and 1 in box
    second = [box[0], box[1]]
    for name, ranks in (("first", first), ("second", second)):
        ts = [make(torch.float32, (1000,), gen) for _ in range(2)]
        want = O.reduce_copy([words(t) for t in ts], comm.dtype_code(torch.float32), comm.op_code(ReduceOp.SUM))
        wait_all([b.allreduce([t], dist.AllreduceOptions()) for b, t in zip(ranks, ts)])
        for r, t in enumerate(ts):
            same(words(t).ravel(), want, f"{name} group over a shared store, rank {r}")
    print("ok  two successive groups over one HashStore", flush=True)


def one_rank(gen):
    fxb.register()
    dist.init_process_group("flagcx", store=dist.HashStore(), rank=0, world_size=1)
    try:
        assert dist.get_backend() == "flagcx"
        t = make(torch.float32, (100003,), gen)
        keep = t.clone()
        dist.all_reduce(t)
        assert torch.equal(t, keep)
        dist.all_reduce(t, op=ReduceOp.AVG)
        assert torch.equal(t, keep)
        out = [torch.empty_like(t)]
        dist.all_gather(out, t)
        assert torch.equal(out[0], keep)
        flat = torch.empty_like(t)
        dist.all_gather_into_tensor(flat, t)
        dist.reduce_scatter_tensor(out[0], flat)
        dist.broadcast(t, 0)
        dist.all_to_all_single(flat, t)
        assert torch.equal(flat, keep) and torch.equal(out[0], keep)
        w = dist.all_reduce(t, async_op=True)
        w.wait()
        assert w.is_completed() or torch.cuda.synchronize() is None
        dist.barrier()
        torch.cuda.synchronize()
        assert torch.equal(t, keep)
        # batched point-to-point (a coalescing bracket) and the coalescing manager around collectives
        box = torch.empty_like(t)
        for w in dist.batch_isend_irecv([dist.P2POp(dist.isend, t, 0), dist.P2POp(dist.irecv, box, 0)]):
            w.wait()
        a, b2 = t.clone(), t[:77].clone()
        with dist._coalescing_manager(device=torch.device("cuda")):
            dist.all_reduce(a)
            dist.all_reduce(b2)
        torch.cuda.synchronize()
        assert torch.equal(box, keep) and torch.equal(a, keep) and torch.equal(b2, keep[:77])
        # DistributedDataParallel: parameter broadcast, shape check and gradient buckets all go through the backend
        torch.manual_seed(0)
        model = torch.nn.Sequential(torch.nn.Linear(64, 128), torch.nn.ReLU(), torch.nn.Linear(128, 8)).cuda()
        ddp = torch.nn.parallel.DistributedDataParallel(model, device_ids=[0])
        x = torch.randn(32, 64, device="cuda")
        ddp(x).square().mean().backward()
        grads = [p.grad.clone() for p in model.parameters()]
        model.zero_grad()
        model(x).square().mean().backward()
        assert all(torch.equal(g, p.grad) for g, p in zip(grads, model.parameters())), "DDP gradients differ"
    finally:
        dist.destroy_process_group()
    print("ok  init_process_group('flagcx'), world_size 1, module API and DistributedDataParallel", flush=True)


def main():
    assert torch.cuda.is_available(), "no GPU visible to torch"
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda").manual_seed(5)
    with open("/proc/self/maps") as f:
        print("HIP runtime in this process:", sorted({ln.split()[-1] for ln in f if "libamdhip64" in ln}), flush=True)
    simulated(4, gen)
    simulated(8, gen)
    two_groups_over_one_store(gen)
    one_rank(gen)
    print("torch backend ok", flush=True)


if __name__ == "__main__":
    main()
