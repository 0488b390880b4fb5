"""The native collective performance tool (flagcx_amd/lib/fx_collperf): every
collective it knows, with its own result check switched on, for 8 ranks and
for more ranks than a slice descriptor has input slots."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

TOOL = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "flagcx_amd", "lib", "fx_collperf")
COLLECTIVES = ["allreduce", "reduce", "reducescatter", "allgather", "broadcast", "gather", "scatter", "alltoall",
               "alltoallv", "sendrecv"]


def run(*args):
    p = subprocess.run([TOOL, *args], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, f"{' '.join(args)}\n{p.stdout}\n{p.stderr}"
    return p.stdout


@pytest.mark.parametrize("coll", COLLECTIVES)
def test_tool_checks_its_own_results(coll):
    assert os.path.exists(TOOL), "fx_collperf is not built (python -m flagcx_amd.build)"
    for extra in (["-N", "8"], ["-N", "12", "-r", "7", "-d", "int32", "-o", "max"], ["-N", "3", "-d", "double", "-O", "ring"]):
        out = run(coll, "-b", "4K", "-e", "3M", "-f", "27", "-w", "1", "-n", "3", "-c", "1", *extra)
        assert "# check: every rank's result as expected" in out, out
        lines = [ln for ln in out.splitlines() if ln.startswith("Comm size:")]
        assert len(lines) == 3 and all("Bus bandwidth" in ln and "on the device" in ln for ln in lines), out


@pytest.mark.parametrize("coll", ["allreduce", "reducescatter", "allgather", "alltoallv", "sendrecv"])
def test_a_thread_and_a_stream_per_rank(coll):
    """-T 1: every rank's calls come from its own host thread on its own stream
    and block until all ranks have posted, the way separate processes behave."""
    out = run(coll, "-b", "64K", "-e", "4M", "-f", "8", "-w", "2", "-n", "10", "-c", "1", "-T", "1", "-N", "4")
    assert "a host thread and a stream per rank" in out and "# check: every rank's result as expected" in out, out


def test_tool_moves_narrow_types_and_reports_what_it_cannot_check():
    out = run("allgather", "-b", "64K", "-e", "64K", "-d", "bfloat16", "-c", "1", "-n", "2")
    assert "# check: every rank's result as expected" in out
    out = run("allreduce", "-b", "64K", "-e", "64K", "-d", "half", "-c", "1", "-n", "2")
    assert "no check for this datatype / op" in out
    out = run("allreduce", "-b", "1M", "-e", "1M", "-d", "bfloat16", "-a", "element", "-n", "3")
    assert len([ln for ln in out.splitlines() if ln.startswith("Comm size:")]) == 1
    bad = subprocess.run([TOOL, "allreduce", "-N", "65"], capture_output=True, text=True, timeout=60)
    assert bad.returncode == 1 and "bad value for -N" in bad.stderr
    bad = subprocess.run([TOOL, "allsomething"], capture_output=True, text=True, timeout=60)
    assert bad.returncode == 1 and "unknown collective" in bad.stderr
