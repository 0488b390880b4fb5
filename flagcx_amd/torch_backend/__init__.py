"""torch.distributed backend "flagcx" over libflagcx_amd.so (fx_c10d.cpp), the
counterpart of the reference's torch plugin (plugin/torch/flagcx/__init__.py
registers its backend under the same name).

    import flagcx_amd.torch_backend as fxb
    fxb.register()                                   # once per process
    torch.distributed.init_process_group("flagcx", store=..., rank=0, world_size=1)

With simulated ranks (every rank of the group in this process, one GPU) build one
backend object per rank from a shared store and post every rank's call before
waiting on any of the returned Work objects:

    store = torch.distributed.HashStore()
    ranks = [fxb.new_backend(store, r, n) for r in range(n)]
    works = [b.allreduce([t]) for b, t in zip(ranks, tensors)]
    for w in works: w.wait()
"""
import importlib.util
import os

_ext = None


def extension():
    """The compiled module; raises if it has not been built."""
    global _ext
    if _ext is None:
        import torch  # noqa: F401  (its libraries must be loaded first)
        libdir = os.environ.get("FLAGCX_AMD_LIB_DIR") or os.path.join(os.path.dirname(os.path.dirname(
            os.path.abspath(__file__))), "lib")
        path = os.path.join(libdir, "fx_c10d.so")
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: build it with python -m flagcx_amd.torch_backend.build")
        spec = importlib.util.spec_from_file_location("fx_c10d", path)
        _ext = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(_ext)
    return _ext


def new_backend(store, rank, size):
    """One rank's c10d backend object (a torch.distributed Backend)."""
    return extension().create_backend(store, rank, size)


def _create(store, rank, size, timeout):
    return new_backend(store, rank, size)


def register(name="flagcx"):
    """Make `name` usable in torch.distributed.init_process_group for GPU tensors."""
    import torch.distributed as dist
    extension()
    dist.Backend.register_backend(name, _create, devices=["cuda"])
