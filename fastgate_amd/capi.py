"""ctypes binding of libfastgate's C ABI (include/fastgate.h).

This is the thin, allocation-free route to the kernels: raw device pointers, sizes and a HIP
stream handle.  It is what the C-ABI tests and the benchmark call; the pybind11 module
`speedgate` reaches the same entry points from C++.  There is no fallback: if the shared
library is missing, loading raises.
"""
from __future__ import annotations

import ctypes
from pathlib import Path

_PKG = Path(__file__).resolve().parent
LIB_PATH = _PKG / "libfastgate.so"

FG_OK = 0
FG_ERR_INVALID_ARG = -1
FG_ERR_ALIGN128 = -2
FG_ERR_WORKSPACE = -3
FG_ERR_LAUNCH = -4
FG_ERR_UNSUPPORTED = -5
FG_ERR_SCRATCH_LIMIT = -6
FG_STATIC_SCRATCH_BYTES = 65536 + 3145728 + 524288 + (8 << 20)

FG_W_KN = 0
FG_W_NK = 1

FG_KERNEL_AUTO = 0
FG_KERNEL_NK_DOT2 = 1
FG_KERNEL_KN_DOT2 = 3
FG_KERNEL_KN_MFMA = 4
FG_KERNEL_NK_MFMA4 = 5
FG_KERNEL_NK_MFMA_R = 8
FG_ACT_NONE, FG_ACT_RELU, FG_ACT_GELU, FG_ACT_GELU_TANH, FG_ACT_SILU = range(5)
ACT_IDS = {"none": 0, "relu": 1, "gelu": 2, "gelu_tanh": 3, "silu": 4}
KERNEL_NAMES = {1: "nk_dot2", 3: "kn_dot2", 4: "kn_mfma", 5: "nk_mfma4", 8: "nk_mfma_r"}

# Every symbol include/fastgate.h declares.
EXPORTS = (
    "fg_gemm_f16",
    "fg_gemm_f16_planned",
    "fg_gemm_f16_pitched",
    "fg_gemm_f16_static",
    "fg_gemm_f16_bias_act",
    "fg_plan",
    "fg_workspace_bytes",
    "fg_workspace_header_bytes",
    "fg_workspace_init",
    "fg_set_compute_units",
    "fg_compute_units",
    "fg_use_device_compute_units",
    "fg_gemv_w8a16",
    "fg_gemv_w4a16",
    "fg_gemv_i8i8_i32",
    "fg_dequant_i32_f16",
    "fg_stream_read",
    "fg_stream_read_sink_bytes",
    "fg_strerror",
    "fg_version",
)


class Plan(ctypes.Structure):
    """fg_plan_t"""

    _fields_ = [
        ("kernel", ctypes.c_int),
        ("splitk", ctypes.c_int),
        ("fused", ctypes.c_int),
        ("tile_n", ctypes.c_int),
        ("m_block", ctypes.c_int),
        ("waves", ctypes.c_int),
        ("unroll", ctypes.c_int),
        ("stream_w", ctypes.c_int),
        ("stagger", ctypes.c_int),
        ("band", ctypes.c_int),
        ("grid_x", ctypes.c_int),
        ("grid_y", ctypes.c_int),
        ("grid_z", ctypes.c_int),
        ("block", ctypes.c_int),
        ("workspace_bytes", ctypes.c_size_t),
    ]

    def as_dict(self) -> dict:
        d = {name: getattr(self, name) for name, _ in self._fields_}
        d["kernel_name"] = KERNEL_NAMES.get(self.kernel, "?")
        return d


class FastgateError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        super().__init__("%s: %s (status %d)" % (where, strerror(status), status))


_lib = None


def lib() -> ctypes.CDLL:
    """Load libfastgate.so from the package directory (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise FileNotFoundError(
                "%s is missing: build it with `python -m fastgate_amd.build`" % LIB_PATH)
        L = ctypes.CDLL(str(LIB_PATH))
        vp, ci, cf, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
        pp = ctypes.POINTER(Plan)
        L.fg_gemm_f16.restype = ci
        L.fg_gemm_f16.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, ci, vp, sz, vp]
        L.fg_gemm_f16_pitched.restype = ci
        L.fg_gemm_f16_pitched.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, ci, vp, sz, vp]
        L.fg_gemm_f16_static.restype = ci
        L.fg_gemm_f16_static.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
        L.fg_gemm_f16_planned.restype = ci
        L.fg_gemm_f16_planned.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, pp, vp, sz, vp]
        L.fg_gemm_f16_bias_act.restype = ci
        L.fg_gemm_f16_bias_act.argtypes = [vp, vp, vp, ci, vp, ci, ci, ci, ci, ci, pp, vp, sz, vp]
        L.fg_plan.restype = ci
        L.fg_plan.argtypes = [ci, ci, ci, ci, ci, pp]
        L.fg_workspace_bytes.restype = sz
        L.fg_workspace_bytes.argtypes = [ci, ci, ci, ci, ci]
        L.fg_workspace_header_bytes.restype = sz
        L.fg_workspace_header_bytes.argtypes = []
        L.fg_workspace_init.restype = ci
        L.fg_workspace_init.argtypes = [vp, sz, vp]
        L.fg_set_compute_units.restype = ci
        L.fg_set_compute_units.argtypes = [ci]
        L.fg_compute_units.restype = ci
        L.fg_compute_units.argtypes = []
        L.fg_use_device_compute_units.restype = ci
        L.fg_use_device_compute_units.argtypes = []
        L.fg_gemv_w8a16.restype = ci
        L.fg_gemv_w8a16.argtypes = [vp, vp, vp, cf, cf, vp, ci, ci, ci, vp]
        L.fg_gemv_w4a16.restype = ci
        L.fg_gemv_w4a16.argtypes = [vp, vp, vp, cf, cf, vp, ci, ci, ci, vp]
        L.fg_gemv_i8i8_i32.restype = ci
        L.fg_gemv_i8i8_i32.argtypes = [vp, vp, vp, ci, ci, ci, vp]
        L.fg_dequant_i32_f16.restype = ci
        L.fg_dequant_i32_f16.argtypes = [vp, vp, cf, vp, ci, ci, vp]
        L.fg_stream_read.restype = ci
        L.fg_stream_read.argtypes = [vp, sz, vp, vp]
        L.fg_stream_read_sink_bytes.restype = sz
        L.fg_stream_read_sink_bytes.argtypes = []
        L.fg_strerror.restype = ctypes.c_char_p
        L.fg_strerror.argtypes = [ci]
        L.fg_version.restype = ci
        L.fg_version.argtypes = []
        _lib = L
    return _lib


def strerror(status: int) -> str:
    return lib().fg_strerror(int(status)).decode()


def check(status: int, where: str) -> None:
    if status != FG_OK:
        raise FastgateError(status, where)


def plan(M: int, N: int, K: int, w_layout: int, splitk: int = 0) -> Plan:
    p = Plan()
    check(lib().fg_plan(M, N, K, w_layout, splitk, ctypes.byref(p)), "fg_plan")
    return p


def workspace_bytes(M: int, N: int, K: int, w_layout: int, splitk: int = 0) -> int:
    return int(lib().fg_workspace_bytes(M, N, K, w_layout, splitk))
