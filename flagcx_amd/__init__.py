"""MI355X-native reduce / slice / pack path behind FlagCX's plugin boundary.

The product is the shared libraries under ``flagcx_amd/lib`` (built from
``flagcx_amd/csrc`` by ``python -m flagcx_amd.build``).  This package is the thin
ctypes glue the tests and the benchmark use to call their C ABI; it contains no
arithmetic and has no CPU fallback: a missing library is an ImportError.
"""
from . import _native  # noqa: F401
from ._native import (DT_BF16, DT_FP16, DT_FP32, DT_INT32, DTYPE_SIZE, NP_DTYPE,
                      OP_MAX, OP_MIN, OP_PROD, OP_SUM, FlagcxError, check, lib)

__all__ = ["lib", "check", "FlagcxError", "DT_INT32", "DT_FP16", "DT_FP32",
           "DT_BF16", "OP_SUM", "OP_PROD", "OP_MAX", "OP_MIN", "DTYPE_SIZE",
           "NP_DTYPE"]
