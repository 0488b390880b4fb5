"""Compile the HIP libraries in-tree: ``python -m flagcx_amd.build``."""
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def build(jobs=8, clean=False):
    if clean:
        subprocess.check_call(["make", "-C", CSRC, "clean"])
    subprocess.check_call(["make", "-C", CSRC, f"-j{jobs}", "all"])


if __name__ == "__main__":
    build(clean="--clean" in sys.argv)
