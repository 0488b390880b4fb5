"""The committed fixtures (tests/golden/golden.json) must be what the oracle and
the input generator produce on THIS machine: guards against drift between the
container that wrote them and the box that runs the GPU tests."""
import json
import os

import numpy as np
import pytest

from flagcx_amd import _native as N
from oracle import fx_oracle as O
from tests.golden import workloads as W

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "golden.json")))


@pytest.fixture(scope="module", autouse=True)
def _threads():
    O.lib.oracle_set_threads(8)
    yield
    O.lib.oracle_set_threads(1)


def _check(entry, ins, out):
    if "inputs_sha256" in entry:
        assert [W.digest(a) for a in ins] == entry["inputs_sha256"], "seeded inputs differ on this machine"
    assert W.probe(out) == entry["out_probe"]
    assert W.digest(out) == entry["out_sha256"]


def test_cfg1_full_size():
    c = W.CFG1
    ins = W.inputs(c["dtype"], c["k"], c["n"], c["dist"], c["seed"])
    _check(GOLDEN["cfg1_fp32_sum_2x16777216"], ins, O.reduce_copy(ins, c["dtype"], N.OP_SUM))


def test_cfg2_and_cfg5_reduced():
    c = W.CFG2
    ins = W.inputs(c["dtype"], c["k"], c["n"] // 16, c["dist"], c["seed"])
    _check(GOLDEN["cfg2_bf16_sum_8x2097152"], ins, O.reduce_copy(ins, c["dtype"], N.OP_SUM))
    c = W.CFG5
    ins = W.inputs(c["dtype"], c["k"], 4_194_304, c["dist"], c["seed"])
    _check(GOLDEN["cfg5_bf16_sum_8x4194304"], ins, O.reduce_copy(ins, c["dtype"], N.OP_SUM))
    # the reduced case is a prefix of the full one
    full = GOLDEN["cfg5_bf16_sum_8x268435456"]
    assert full["out_probe"][:2] == GOLDEN["cfg5_bf16_sum_8x4194304"]["out_probe"][:2]


@pytest.mark.parametrize("dtype", list(W.CFG3["dists"]))
def test_cfg3_every_case_up_to_16MiB(dtype):
    es = N.DTYPE_SIZE[dtype]
    big = W.cfg3_inputs(dtype, (1 << 24) // es)
    for oname, op in W.OPS.items():
        for lg in range(10, 25):
            n = (1 << lg) // es
            out = O.reduce_copy([a[:n] for a in big], dtype, op)
            _check(GOLDEN["cfg3"][f"{W.DTYPE_NAMES[dtype]}_{oname}_{1 << lg}"], None, out)


def test_cfg4_layout_and_digests():
    e = GOLDEN["cfg4_alltoallv_pack_unpack"]
    counts, sd, slen, rd, rlen = W.cfg4_layout()
    assert (counts, sd, slen, rd, rlen) == (e["counts"], e["sdispls"], e["send_len"], e["rdispls"], e["recv_len"])
    assert len(counts) == 8 and all(1 <= c <= 4_194_304 for c in counts)
    for displs, total in ((sd, slen), (rd, rlen)):          # segments do not overlap
        segs = sorted(zip(displs, counts))
        assert all(a + c <= b for (a, c), (b, _) in zip(segs, segs[1:])) and segs[-1][0] + segs[-1][1] <= total
    send = W.inputs(N.DT_FP32, 1, slen, (0, -1.0, 1.0), W.CFG4["seed"])[0]
    assert W.digest(send) == e["send_sha256"]
    packed = O.pack(send, counts, sd)
    assert W.digest(packed) == e["packed_sha256"]
    assert W.digest(O.unpack(np.zeros(rlen, np.float32), packed, counts, rd)) == e["unpacked_sha256"]


def test_every_type_and_op_small_matrix():
    for dname, dtype in W.ALL_DTYPES.items():
        ins = W.matrix_inputs(dtype)
        for oname, op in W.ALL_OPS.items():
            _check(GOLDEN["matrix"][f"{dname}_{oname}"], ins, O.reduce_copy(ins, dtype, op))


def test_reference_schedules_on_one_case():
    e = GOLDEN["schedules_fp32_sum_5x1003"]
    sends = W.inputs(N.DT_FP32, 5, 1003, (0, -1000.0, 1000.0), 6, 1)
    assert [W.digest(a) for a in sends] == e["inputs_sha256"]
    got = {"ring": O.ring_allreduce(sends, N.DT_FP32, N.OP_SUM)[0], "tree_root2": O.tree_reduce(sends, 2, N.DT_FP32, N.OP_SUM),
           "host": O.bootstrap_allreduce(sends, N.DT_FP32, N.OP_SUM)[0], "rank": O.reduce_copy(sends, N.DT_FP32, N.OP_SUM)}
    assert {k: W.digest(v) for k, v in got.items()} == {k: e[k] for k in got}
    assert len({e[k] for k in got}) == 4, "the four schedules are expected to round differently on this case"
