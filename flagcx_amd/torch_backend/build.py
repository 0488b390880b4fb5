"""Compiles the torch.distributed backend module (fx_c10d.cpp) against the
installed torch and the in-tree libflagcx_amd.so.  Host code only: the module
launches nothing itself."""
import os
import subprocess
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIBDIR = os.path.join(ROOT, "flagcx_amd", "lib")
OUT = os.path.join(LIBDIR, "fx_c10d.so")


def build(verbose=False):
    import torch
    from torch.utils import cpp_extension as ext
    import pybind11
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    inc = ext.include_paths("cpu") + [pybind11.get_include(), sysconfig.get_paths()["include"],
                                      os.path.join(ROOT, "include"), "/opt/rocm/include"]
    cmd = [hipcc, "-x", "c++", "-std=c++17", "-O2", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall",
           "-Wno-unused-function", "-Wno-deprecated-declarations",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=fx_c10d",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    cmd += [f"-I{p}" for p in inc]
    cmd += [os.path.join(HERE, "fx_c10d.cpp"), "-o", OUT]
    for d in ext.library_paths("cpu"):
        cmd += [f"-L{d}"]
    cmd += ["-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            f"-L{LIBDIR}", "-lflagcx_amd", "-L/opt/rocm/lib", "-lamdhip64", "-ldl", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
