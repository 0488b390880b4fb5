"""Every cache policy a launch can carry gives the same bits.  The policy is
chosen per launch from its sizes, or forced for a whole process through the
environment (read once), so each forced policy runs tests/policy_client.py in a
process of its own: streaming loads and stores, ordinary loads for every input,
results left in the cache, both, and the size threshold for ordinary loads."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("env", [{"FX_CACHE_POLICY": "stream"}, {"FX_CACHE_POLICY": "keep"},
                                 {"FX_CACHE_POLICY": "keep-loads"}, {"FX_CACHE_POLICY": "keep-stores"},
                                 {"FX_TEMPORAL_MAX_BYTES": str(16 << 20)}, {}],
                         ids=["stream", "keep", "keep-loads", "keep-stores", "temporal-16MiB", "by-rule"])
def test_every_cache_policy_gives_the_oracles_bits(dev, env):
    base = {k: v for k, v in os.environ.items() if k not in ("FX_CACHE_POLICY", "FX_TEMPORAL_MAX_BYTES")}
    full = dict(base, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""), **env)
    r = subprocess.run([sys.executable, "-u", os.path.join(ROOT, "tests", "policy_client.py")], cwd=ROOT, env=full,
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "policy client ok" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]
