#!/usr/bin/env python3
"""Writes tests/golden/golden.json: digests of the CPU oracle's outputs on the
seeded inputs of every configuration of BASELINE.json.

    python tests/golden/make_golden.py [--full]

The reference holds no vectors for random data (its tests use closed forms), so
these fixtures are produced by this repository's own oracle after it has been
pinned by tests/test_cpu_oracle.py; they exist so that (a) the oracle and the
input generator cannot drift silently between machines or commits and (b) the
GPU result at FULL size can be compared bit for bit without shipping gigabytes.
--full also covers the two full-size cases (needs ~10 GiB of host memory).
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

from flagcx_amd import _native as N  # noqa: E402
from oracle import fx_oracle as O  # noqa: E402
from tests.golden import workloads as W  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden.json")


def entry(ins, out):
    return {"inputs_sha256": [W.digest(a) for a in ins], "out_sha256": W.digest(out), "out_probe": W.probe(out)}


def main():
    full = "--full" in sys.argv
    O.lib.oracle_set_threads(8)
    g = json.load(open(OUT)) if os.path.exists(OUT) else {}

    c = W.CFG1
    ins = W.inputs(c["dtype"], c["k"], c["n"], c["dist"], c["seed"])
    g["cfg1_fp32_sum_2x16777216"] = entry(ins, O.reduce_copy(ins, c["dtype"], N.OP_SUM))

    # cfg2 at 1/16 scale (same slicing arithmetic, 2,097,152 elements per rank) and, with --full, at full scale
    c = W.CFG2
    for label, n in (("cfg2_bf16_sum_8x2097152", c["n"] // 16),) + ((("cfg2_bf16_sum_8x33554432", c["n"]),) if full else ()):
        ins = W.inputs(c["dtype"], c["k"], n, c["dist"], c["seed"])
        g[label] = entry(ins, O.reduce_copy(ins, c["dtype"], N.OP_SUM))

    # cfg3: every op x dtype, sizes 1 KiB .. 16 MiB per input (larger sizes are checked against the oracle live)
    c = W.CFG3
    g["cfg3"] = {}
    for dtype in c["dists"]:
        es = N.DTYPE_SIZE[dtype]
        big = W.cfg3_inputs(dtype, (1 << 24) // es)
        for oname, op in W.OPS.items():
            for lg in range(10, 25):
                n = (1 << lg) // es
                ins = [a[:n] for a in big]
                out = O.reduce_copy(ins, dtype, op)
                g["cfg3"][f"{W.DTYPE_NAMES[dtype]}_{oname}_{1 << lg}"] = {"out_sha256": W.digest(out),
                                                                          "out_probe": W.probe(out)}

    counts, sd, slen, rd, rlen = W.cfg4_layout()
    send = W.inputs(N.DT_FP32, 1, slen, (0, -1.0, 1.0), W.CFG4["seed"])[0]
    packed = O.pack(send, counts, sd)
    recv = O.unpack(np.zeros(rlen, np.float32), packed, counts, rd)
    g["cfg4_alltoallv_pack_unpack"] = {"counts": counts, "sdispls": sd, "send_len": slen, "rdispls": rd,
                                       "recv_len": rlen, "send_sha256": W.digest(send),
                                       "packed_sha256": W.digest(packed), "unpacked_sha256": W.digest(recv)}

    # every element type x every op at a small size, plus the three reference schedules on one fp32 case
    g["matrix"] = {}
    for dname, dtype in W.ALL_DTYPES.items():
        ins = W.matrix_inputs(dtype)
        for oname, op in W.ALL_OPS.items():
            g["matrix"][f"{dname}_{oname}"] = entry(ins, O.reduce_copy(ins, dtype, op))
    sends = W.inputs(N.DT_FP32, 5, 1003, (0, -1000.0, 1000.0), 6, 1)
    g["schedules_fp32_sum_5x1003"] = {
        "inputs_sha256": [W.digest(a) for a in sends],
        "ring": W.digest(O.ring_allreduce(sends, N.DT_FP32, N.OP_SUM)[0]),
        "tree_root2": W.digest(O.tree_reduce(sends, 2, N.DT_FP32, N.OP_SUM)),
        "host": W.digest(O.bootstrap_allreduce(sends, N.DT_FP32, N.OP_SUM)[0]),
        "rank": W.digest(O.reduce_copy(sends, N.DT_FP32, N.OP_SUM)),
    }

    c = W.CFG5
    for label, n in (("cfg5_bf16_sum_8x4194304", 4_194_304),) + ((("cfg5_bf16_sum_8x268435456", c["n"]),) if full else ()):
        ins = W.inputs(c["dtype"], c["k"], n, c["dist"], c["seed"])
        g[label] = entry(ins, O.reduce_copy(ins, c["dtype"], N.OP_SUM))

    json.dump(g, open(OUT, "w"), indent=1, sort_keys=True)
    print(f"wrote {OUT}: {len(g)} top-level entries, {len(g['cfg3'])} cfg3 cases")


if __name__ == "__main__":
    main()
