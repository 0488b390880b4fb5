"""A PyTorch-ROCm caller of the library, run as a process of its own by
tests/test_gpu_torch.py: torch is imported first, so the HIP runtime inside the
process is the one torch ships and the library binds to it (same soname).

It does what the reference's torch backend does for the calls of this path
(plugin/torch/flagcx/src/backend_flagcx.cpp: tensor.data_ptr(), element count,
dtype and ReduceOp mapped to the FlagCX enums, the current stream wrapped by the
device adaptor's streamCopy): tensors of n simulated ranks live on cuda:0, the
collectives run on torch's streams, and the results are read back with torch
and compared bit for bit with the CPU oracle.  Prints one line per case and
"torch client ok" at the end; any mismatch raises."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import torch                                    # noqa: E402  (first on purpose)
import numpy as np
from torch.distributed import ReduceOp

from flagcx_amd import _native as N
from flagcx_amd import kernels as K
from flagcx_amd import comm
from oracle import fx_oracle as O

BITS = {torch.bfloat16: torch.int16, torch.float16: torch.int16, torch.float32: torch.int32, torch.int32: torch.int32,
        torch.int64: torch.int64, torch.float64: torch.int64, torch.uint8: torch.uint8, torch.int8: torch.int8}


def host_words(t):
    """The tensor's bytes as the numpy array the oracle takes for its dtype."""
    dt = comm.dtype_code(t.dtype)
    raw = t.detach().contiguous().view(BITS[t.dtype]).cpu().numpy()
    return raw.view(N.NP_DTYPE[dt])


def make(dtype, n, gen):
    if dtype.is_floating_point:
        return (torch.randn(n, device="cuda", generator=gen, dtype=torch.float32) * 3).to(dtype)
    info = torch.iinfo(dtype)
    return torch.randint(info.min, info.max, (n,), device="cuda", generator=gen, dtype=dtype)


def check(got, want, what):
    g, w = np.ascontiguousarray(got).view(np.uint8), np.ascontiguousarray(want).view(np.uint8)
    if not np.array_equal(g, w):
        bad = np.flatnonzero(g != w)
        raise SystemExit(f"{what}: {bad.size} bytes differ, first at {bad[0]}")
    print(f"ok  {what}", flush=True)


def main():
    assert torch.cuda.is_available(), "no GPU visible to torch"
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda").manual_seed(11)
    with open("/proc/self/maps") as f:
        print("HIP runtime in this process:", sorted({ln.split()[-1] for ln in f if "libamdhip64" in ln}), flush=True)
    nranks = 4
    ranks = comm.join(nranks)
    side = torch.cuda.Stream()

    # ---- the kernel layer on raw torch pointers and torch's current stream ----
    for dtype, op in [(torch.bfloat16, ReduceOp.SUM), (torch.float32, ReduceOp.PRODUCT), (torch.int32, ReduceOp.MAX)]:
        n = 1_000_003
        ins = [make(dtype, n, gen) for _ in range(5)]
        out = torch.empty_like(ins[0])
        dt, rop = comm.dtype_code(dtype), comm.op_code(op)
        print(f"run reduce_copy {dtype} {op} n={n}", flush=True)
        rc = K.reduce_copy(out.data_ptr(), [t.data_ptr() for t in ins], n, dt, rop, 0,
                           torch.cuda.current_stream().cuda_stream)
        assert rc == N.SUCCESS, rc
        torch.cuda.synchronize()
        check(host_words(out), O.reduce_copy([host_words(t) for t in ins], dt, rop), f"reduce_copy {dtype} {op}")

    # ---- FlagCX-named collectives, one call per simulated rank, on torch streams ----
    for dtype, op, stream in [(torch.bfloat16, ReduceOp.SUM, side), (torch.float16, ReduceOp.AVG, side),
                              (torch.float32, ReduceOp.SUM, torch.cuda.current_stream()),
                              (torch.int64, ReduceOp.MIN, side), (torch.float64, ReduceOp.SUM, side)]:
        n = 262_147
        sends = [make(dtype, n, gen) for _ in range(nranks)]
        recvs = [torch.empty_like(s) for s in sends]
        dt, rop = comm.dtype_code(dtype), comm.op_code(op)
        print(f"run allreduce {dtype} {op} n={n}", flush=True)
        stream.wait_stream(torch.cuda.current_stream())          # the fills above ran on the current stream
        fs = comm.borrow_stream(stream)
        for r in range(nranks):
            ranks[r].all_reduce(sends[r].data_ptr(), recvs[r].data_ptr(), n, dt, rop, fs)
        torch.cuda.current_stream().wait_stream(stream)
        want = O.reduce_copy([host_words(s) for s in sends], dt, rop)
        for r in range(nranks):
            check(host_words(recvs[r]), want, f"allreduce {dtype} {op} rank {r}")
        comm.return_stream(fs)

    # in place, then reduce-scatter + all-gather give the same words as the all-reduce
    n = nranks * 65_536
    sends = [make(torch.bfloat16, n, gen) for _ in range(nranks)]
    want = O.reduce_copy([host_words(s) for s in sends], N.DT_BF16, N.OP_SUM)
    parts = [torch.empty(n // nranks, device="cuda", dtype=torch.bfloat16) for _ in range(nranks)]
    full = [torch.empty(n, device="cuda", dtype=torch.bfloat16) for _ in range(nranks)]
    fs = comm.borrow_stream(torch.cuda.current_stream())
    print("run reducescatter + allgather bf16", flush=True)
    for r in range(nranks):
        ranks[r].reduce_scatter(sends[r].data_ptr(), parts[r].data_ptr(), n // nranks, N.DT_BF16, N.OP_SUM, fs)
    for r in range(nranks):
        ranks[r].all_gather(parts[r].data_ptr(), full[r].data_ptr(), n // nranks, N.DT_BF16, fs)
    for r in range(nranks):
        ranks[r].all_reduce(sends[r].data_ptr(), sends[r].data_ptr(), n, N.DT_BF16, N.OP_SUM, fs)
    torch.cuda.synchronize()
    for r in range(nranks):
        check(host_words(full[r]), want, f"reducescatter+allgather rank {r}")
        check(host_words(sends[r]), want, f"allreduce in place rank {r}")
    comm.return_stream(fs)
    for r in ranks:
        r.close()
    print("torch client ok", flush=True)


if __name__ == "__main__":
    sys.exit(main())
