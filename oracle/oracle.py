"""numpy front end of the C oracle (oracle/fg_oracle.c) plus a restatement of the reference's
operator conventions: which argument is the weight, which dimension is N, which entry points
overwrite C and which accumulate into it, and which arguments they reject.

TEST INFRASTRUCTURE ONLY.  Nothing under fastgate_amd/ imports this module.

Reference citations are relative to the root of chanzhennan/Fastgate.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "libfg_oracle.so"
_lib = None

W_KN, W_NK = 0, 1


def build(force: bool = False) -> Path:
    """Compile fg_oracle.c with gcc (a second or two)."""
    src = _HERE / "fg_oracle.c"
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < src.stat().st_mtime:
        _LIB_PATH.parent.mkdir(exist_ok=True)
        subprocess.run(
            ["gcc", "-O2", "-ffp-contract=off", "-fPIC", "-Wall", "-Wextra", "-shared",
             "-o", str(_LIB_PATH), str(src), "-lm"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()  # compiles only when the library is missing or older than its source
        L = ctypes.CDLL(str(_LIB_PATH))
        vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L.fg_oracle_h2f.restype = ctypes.c_float
        L.fg_oracle_h2f.argtypes = [ctypes.c_uint16]
        L.fg_oracle_f2h.restype = ctypes.c_uint16
        L.fg_oracle_f2h.argtypes = [ctypes.c_float]
        L.fg_oracle_d2h.restype = ctypes.c_uint16
        L.fg_oracle_d2h.argtypes = [ctypes.c_double]
        L.fg_oracle_gemm_f16.restype = None
        L.fg_oracle_gemm_f16.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
        L.fg_oracle_gemm_f16_f64.restype = None
        L.fg_oracle_gemm_f16_f64.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
        L.fg_oracle_gemv_w8a16.restype = None
        L.fg_oracle_gemv_w8a16.argtypes = [vp, vp, vp, cf, cf, vp, vp, ci, ci, ci]
        L.fg_oracle_gemv_w4a16.restype = None
        L.fg_oracle_gemv_w4a16.argtypes = [vp, vp, vp, cf, cf, vp, vp, ci, ci, ci]
        L.fg_oracle_gemv_i8i8_i32.restype = ci
        L.fg_oracle_gemv_i8i8_i32.argtypes = [vp, vp, vp, ci, ci, ci]
        L.fg_oracle_dequant_i32_f16.restype = None
        L.fg_oracle_dequant_i32_f16.argtypes = [vp, vp, cf, vp, ci, ci]
        L.fg_oracle_bias_act.restype = None
        L.fg_oracle_bias_act.argtypes = [vp, vp, ci, vp, vp, ci, ci]
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


def _f16(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype != np.float16:
        raise TypeError("expected float16, got %s" % a.dtype)
    return a


def h2f(bits: int) -> float:
    return float(lib().fg_oracle_h2f(int(bits) & 0xFFFF))


def f2h(value: float) -> int:
    return int(lib().fg_oracle_f2h(float(np.float32(value))))


def d2h(value: float) -> int:
    return int(lib().fg_oracle_d2h(float(value)))


def gemm_f16(A, W, w_layout: int, C=None, accumulate: bool = False, acc: str = "f32"):
    """C = A·W (or C += A·W).  Returns (C as float16 [M,N], unrounded sums [M,N] in the
    accumulation type, without the accumulate term)."""
    A, W = _f16(A), _f16(W)
    M, K = A.shape
    if w_layout == W_KN:
        if W.shape[0] != K:
            raise ValueError("W[K,N] does not match A[M,K]")
        N = W.shape[1]
    elif w_layout == W_NK:
        if W.shape[1] != K:
            raise ValueError("W[N,K] does not match A[M,K]")
        N = W.shape[0]
    else:
        raise ValueError("w_layout")
    if accumulate:
        if C is None:
            raise ValueError("accumulate needs C")
        out = np.ascontiguousarray(C, dtype=np.float16).reshape(M, N).copy()
    else:
        out = np.zeros((M, N), np.float16)
    if acc == "f32":
        raw = np.zeros((M, N), np.float32)
        row = np.zeros(N, np.float32)
        fn = lib().fg_oracle_gemm_f16
    elif acc == "f64":
        raw = np.zeros((M, N), np.float64)
        row = np.zeros(N, np.float64)
        fn = lib().fg_oracle_gemm_f16_f64
    else:
        raise ValueError("acc")
    fn(_ptr(A), _ptr(W), _ptr(out), _ptr(raw), _ptr(row), M, N, K, int(w_layout), int(bool(accumulate)))
    return out, raw


def gemv_w8a16(Wq, x, scale=None, scalar_scale: float = 1.0, zero_point: float = 0.0):
    """y[m,n] = fp16((Σ_k x[m,k]·(float(Wq[n,k]) − zp))·scalar_scale·scale[n]); returns
    (float16 [M,N], float32 unrounded)."""
    Wq = np.ascontiguousarray(Wq)
    if Wq.dtype != np.int8:
        raise TypeError("Wq must be int8")
    x = _f16(x).reshape(-1, Wq.shape[1])
    M, K = x.shape
    N = Wq.shape[0]
    sc = None if scale is None else _f16(scale).reshape(N)
    y = np.zeros((M, N), np.float16)
    y32 = np.zeros((M, N), np.float32)
    lib().fg_oracle_gemv_w8a16(_ptr(Wq), _ptr(x), _ptr(sc), float(scalar_scale), float(zero_point),
                               _ptr(y), _ptr(y32), M, N, K)
    return y, y32


def gemv_w4a16(Wq4, x, scale=None, scalar_scale: float = 1.0, zero_point: float = 0.0):
    """Wq4 uint8 [N,K/2], two unsigned nibbles per byte (even element in the low nibble):
    y[m,n] = fp16((Σ_k x[m,k]·(float(u4[n,k]) − zp))·scalar_scale·scale[n]); returns
    (float16 [M,N], float32 unrounded)."""
    Wq4 = np.ascontiguousarray(Wq4)
    if Wq4.dtype != np.uint8:
        raise TypeError("Wq4 must be uint8")
    N, K = Wq4.shape[0], Wq4.shape[1] * 2
    x = _f16(x).reshape(-1, K)
    M = x.shape[0]
    sc = None if scale is None else _f16(scale).reshape(N)
    y = np.zeros((M, N), np.float16)
    y32 = np.zeros((M, N), np.float32)
    lib().fg_oracle_gemv_w4a16(_ptr(Wq4), _ptr(x), _ptr(sc), float(scalar_scale), float(zero_point),
                               _ptr(y), _ptr(y32), M, N, K)
    return y, y32


def gemv_i8i8_i32(Wq, xq):
    """acc[m,n] = Σ_k xq[m,k]·Wq[n,k], exact; raises if a sum leaves the int32 range."""
    Wq = np.ascontiguousarray(Wq)
    xq = np.ascontiguousarray(xq)
    if Wq.dtype != np.int8 or xq.dtype != np.int8:
        raise TypeError("int8 expected")
    xq = xq.reshape(-1, Wq.shape[1])
    M, K = xq.shape
    N = Wq.shape[0]
    out = np.zeros((M, N), np.int32)
    if lib().fg_oracle_gemv_i8i8_i32(_ptr(Wq), _ptr(xq), _ptr(out), M, N, K):
        raise OverflowError("int32 overflow in integer dot")
    return out


def dequant_i32_f16(acc, scale, x_scale: float):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    M, N = acc.shape
    sc = None if scale is None else _f16(scale).reshape(N)
    y = np.zeros((M, N), np.float16)
    lib().fg_oracle_dequant_i32_f16(_ptr(acc), _ptr(sc), float(x_scale), _ptr(y), M, N)
    return y


ACTS = {"none": 0, "relu": 1, "gelu": 2, "gelu_tanh": 3, "silu": 4}


def bias_act(raw32, bias=None, act="none"):
    """fp16(act(raw32 + bias[n])) on unrounded fp32 sums [M,N]; returns (float16, float32)."""
    raw = np.ascontiguousarray(raw32, dtype=np.float32)
    M, N = raw.shape
    b = None if bias is None else _f16(bias).reshape(N)
    y = np.zeros((M, N), np.float16)
    y32 = np.zeros((M, N), np.float32)
    lib().fg_oracle_bias_act(_ptr(raw), _ptr(b), int(ACTS[act]), _ptr(y), _ptr(y32), M, N)
    return y, y32


def gemm_bias_act(A, W, w_layout: int, bias=None, act="none"):
    """fp16(act(A·W + bias)): the fp32-accumulate product, then the tail in fp32."""
    _, raw = gemm_f16(A, W, w_layout)
    return bias_act(raw, bias, act)[0]


# ------------------------------------------------------------------------------------------
# The reference's operator surface for this path: name -> (weight layout, C protocol, has bz).
#   "overwrite": the host zeroes C (or the kernel stores plainly) -> C = A·W
#   "accumulate": the host does not zero C and the kernel adds atomically -> C += A·W
# ------------------------------------------------------------------------------------------
GEMM_OPS = {
    # backend/cuda/hk/edgemm.cu
    "edgemm_m8n128k64x4": (W_KN, "overwrite", False),        # :102-156, C.zero_() :141
    "edgemm_m8n128k64x4_amd": (W_KN, "overwrite", False),    # :159-213
    "edgemm_m8n128k64x4_tr_amd": (W_NK, "overwrite", False), # :216-270
    "edgemm_m8n128k64x4_bt": (W_NK, "overwrite", False),     # :274-324, zeroed when BZ>1, plain store else
    "edgemm_m8n256k32x8": (W_KN, "accumulate", False),       # :363-385, no zeroing, always atomics
    # backend/cuda/hk/flatgemm.cu
    "flat_gemm_m8n128k64x4_bz1": (W_KN, "accumulate", True),   # :13-32
    "flat_gemm_m8n256k32x8_bz1": (W_KN, "overwrite", False),   # :34-52, C.zero_() :42
    "flat_gemm_m8n256k64x8": (W_KN, "accumulate", True),       # :55-79
    "flat_gemm_m8n256k32x16": (W_KN, "overwrite", False),      # :81-104, C.zero_() :96
    "flat_gemm_m8n512k32x16": (W_KN, "accumulate", True),      # :106-129
    "flat_gemm_m8n64k128x8": (W_KN, "accumulate", True),       # :132-149
    "flat_gemm_m8n32k256x8": (W_KN, "accumulate", True),       # :152-169
    # backend/cuda/hk/edgemm_tr.cu
    "gemm_m8n128k64x4_bt": (W_NK, "overwrite", False),         # :19-50, C.zero_() :36
    "gemm_m8n32k128x8_bt": (W_NK, "accumulate", False),        # :55-72
    "gemm_m8n64k128x8_bt_exp": (W_NK, "accumulate", True),     # :77-94
    "gemm_m8n32k256x8_bt": (W_NK, "accumulate", False),        # :99-116
    "gemm_m8n32k256x8_bt_bz2": (W_NK, "accumulate", True),     # :122-139
}

ALIGN_MESSAGE = "must be multiple of 128"


def gemm_op(name: str, A, B, C, bz=None):
    """What C holds after `name(A, B, C[, bz])` of the reference, under the fp32-accumulate
    contract.  Raises ValueError where the reference throws std::invalid_argument."""
    layout, protocol, has_bz = GEMM_OPS[name]
    if has_bz != (bz is not None):
        raise TypeError("%s %s a bz argument" % (name, "takes" if has_bz else "does not take"))
    A = _f16(A)
    B = _f16(B)
    M, K = A.shape
    N = B.shape[1] if layout == W_KN else B.shape[0]
    if N % 128 or K % 128:  # e.g. edgemm.cu:107-109
        raise ValueError("K & N " + ALIGN_MESSAGE)
    out, _ = gemm_f16(A, B, layout, C=C, accumulate=(protocol == "accumulate"))
    return out


def fastgemv(mat, vec):
    """fastgemv / fastgemv_tuned (backend/cuda/hk/fastgemv.cu:12-33,63-84): weight FIRST,
    mat[N,K]; vec holds K contiguous elements; result N elements."""
    mat = _f16(mat)
    vec = _f16(vec).reshape(1, mat.shape[1])
    out, _ = gemm_f16(vec, mat, W_NK)
    return out.reshape(-1)


def fastgemv_extend(mat, vecs):
    """fastgemv_extend (hk/fastgemv.cu:86-111): mat[N,K], vecs[M,K] -> res[M,N] row-major
    (store index store_id*N + row, hk/fastgemv.cuh:309)."""
    out, _ = gemm_f16(_f16(vecs), _f16(mat), W_NK)
    return out


def fastgemm(mat, vecs):
    """fastgemm (backend/cuda/czn/fastgemm.cu:13-55): mat[N,K], vecs[M in {1,2},K]; the M=2
    kernel stores the second result at res[row + n] (czn/fastgemm.cuh:390), i.e. [M,N]
    row-major as well."""
    return fastgemv_extend(mat, vecs)


def fastgemv_int8(mat_i8, vec):
    """fastgemv_int8 (hk/fastgemv.cu:35-61): the host passes (zero = 1.0, scale = 0.0) into the
    kernel's (scale, zero_point) parameters, so the effective scale is 1 and zero point 0."""
    y, _ = gemv_w8a16(mat_i8, vec, None, 1.0, 0.0)
    return y.reshape(-1)
