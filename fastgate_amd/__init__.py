"""fastgate_amd — MI355X (gfx950) small-batch GEMM / GEMV operators behind the Fastgate
("SPEEDGATE") operator surface.

    from fastgate_amd import speedgate          # the pybind11 / ATen module
    speedgate.edgemm_m8n128k64x4(A, B, C)       # C[M,N] = A[M,K] @ B[K,N]
    speedgate.edgemm_m8n128k64x4_bt(A, B_t, C)  # C = A @ B_t[N,K].T
    speedgate.fastgemv(W, x, y)                 # weight first, y[N] = W[N,K] @ x[K]

`fastgate_amd.capi` is the ctypes view of the same C ABI (include/fastgate.h).  Both load
native code built in-tree by `python -m fastgate_amd.build`; there is no Python or CPU
fallback, a missing library is an ImportError.
"""
from __future__ import annotations

import importlib

from . import capi  # noqa: F401

__all__ = ["capi", "speedgate", "load_speedgate"]

_speedgate = None


def load_speedgate():
    """Import the pybind11 module (needs torch; loads libfastgate.so next to it)."""
    global _speedgate
    if _speedgate is None:
        import torch  # noqa: F401  (libtorch must be loaded before the extension)

        try:
            _speedgate = importlib.import_module("fastgate_amd.speedgate")
        except ImportError as exc:  # pragma: no cover - build problem, reported loudly
            raise ImportError(
                "fastgate_amd.speedgate is not built (run `python -m fastgate_amd.build`): %s" % exc
            ) from exc
    return _speedgate


def __getattr__(name):
    if name == "speedgate":
        return load_speedgate()
    raise AttributeError(name)
