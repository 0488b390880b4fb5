"""PyTorch-ROCm tensors and streams driving the library, the way the reference's
torch backend does (plugin/torch/flagcx/src/backend_flagcx.cpp: data_ptr(),
numel(), dtype / ReduceOp mapped to FlagCX enums, the current stream wrapped
with streamCopy).  The client runs in a process of its own so that torch's
bundled HIP runtime is loaded there and not under the other GPU tests."""
import importlib.util
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_torch_tensors_and_streams(dev):
    if importlib.util.find_spec("torch") is None:      # looked up, not imported: torch stays out of this process
        pytest.skip("torch is not installed")
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    r = subprocess.run([sys.executable, "-u", os.path.join(ROOT, "tests", "torch_client.py")], cwd=ROOT, env=env,
                       capture_output=True, text=True, timeout=420)
    assert r.returncode == 0 and "torch client ok" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]


def test_torch_distributed_backend(dev):
    """torch.distributed's collectives through the "flagcx" c10d backend module
    (flagcx_amd/torch_backend): 4 and 8 simulated ranks, and a one-rank process group."""
    if importlib.util.find_spec("torch") is None:
        pytest.skip("torch is not installed")
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    r = subprocess.run([sys.executable, "-u", os.path.join(ROOT, "tests", "torch_backend_client.py")], cwd=ROOT, env=env,
                       capture_output=True, text=True, timeout=420)
    assert r.returncode == 0 and "torch backend ok" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]
