"""Writes tests/golden/*.npz: small input/expected-output vectors for the oracle and the GPU
path, computed here with exact integer arithmetic (no floating point, no oracle code).

Every fp16 value is an integer multiple of 2^-24, so a product is an integer multiple of
2^-48 and a dot product is an exact Python int over 2^48.  `round_f16` rounds such a rational
to the nearest fp16 (ties to even) with integer arithmetic only.  The reference
(chanzhennan/Fastgate) holds no vectors for this path; these are ours.

    python tests/golden/make_golden.py      # rewrites the .npz files deterministically
"""
from __future__ import annotations

from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent


def f16_to_int24(bits: int) -> int:
    """fp16 bit pattern -> value * 2^24 as an exact int (finite inputs only)."""
    sign = -1 if bits & 0x8000 else 1
    e = (bits >> 10) & 0x1F
    m = bits & 0x3FF
    assert e != 31, "finite values only"
    if e == 0:
        return sign * m  # subnormal: m * 2^-24
    return sign * ((m | 0x400) << (e - 1))  # (1024+m) * 2^(e-25) * 2^24


def round_f16(num: int, log2den: int) -> int:
    """Nearest fp16 bit pattern (ties to even) of num / 2^log2den."""
    if num == 0:
        return 0
    sign = 0x8000 if num < 0 else 0
    a = abs(num)
    # a / 2^log2den = q * 2^-24 with q rational; work in units of 2^-24 (subnormal spacing)
    # general: find exponent of leading bit
    lead = a.bit_length() - 1 - log2den  # floor(log2(value))
    if lead < -14:
        ulp_log2 = -24
    else:
        ulp_log2 = lead - 10
    # q = value / 2^ulp_log2 = a / 2^(log2den + ulp_log2)
    sh = log2den + ulp_log2
    if sh <= 0:
        q, rem, half = a << (-sh), 0, 1
    else:
        q, rem, half = a >> sh, a & ((1 << sh) - 1), 1 << (sh - 1)
    if rem > half or (rem == half and (q & 1)):
        q += 1
    if lead < -14:
        return sign | q  # q <= 1024; q == 1024 is the smallest normal, encoded identically
    if q == 2048:
        q, lead = 1024, lead + 1
    if lead > 15:
        return sign | 0x7C00
    return sign | ((lead + 15) << 10) | (q & 0x3FF)


def exact_gemm(Abits, Wbits_kn, C0bits=None):
    """Exact A·W for uint16 fp16 bit arrays A[M,K], W[K,N]; returns expected fp16 bits and the
    exact sums as float64 (nearest)."""
    M, K = Abits.shape
    N = Wbits_kn.shape[1]
    a = [[f16_to_int24(int(v)) for v in row] for row in Abits]
    w = [[f16_to_int24(int(v)) for v in row] for row in Wbits_kn]
    out = np.zeros((M, N), np.uint16)
    val = np.zeros((M, N), np.float64)
    for m in range(M):
        for n in range(N):
            s = 0
            for k in range(K):
                s += a[m][k] * w[k][n]
            if C0bits is not None:
                s += f16_to_int24(int(C0bits[m, n])) << 24
            out[m, n] = round_f16(s, 48)
            val[m, n] = s / float(1 << 48)
    return out, val


def main():
    rng = np.random.default_rng(20240611)

    # 1. the stated input distributions: A ~ N(0,1), W ~ N(0,0.02)
    M, K, N = 3, 256, 128
    A = rng.standard_normal((M, K)).astype(np.float16)
    W = (rng.standard_normal((K, N)) * 0.02).astype(np.float16)
    C0 = rng.standard_normal((M, N)).astype(np.float16)
    exp, val = exact_gemm(A.view(np.uint16), W.view(np.uint16))
    exp_acc, _ = exact_gemm(A.view(np.uint16), W.view(np.uint16), C0.view(np.uint16))
    np.savez_compressed(HERE / "gemm_normal.npz", A=A.view(np.uint16), W_kn=W.view(np.uint16),
                        C0=C0.view(np.uint16), expected=exp, expected_accumulate=exp_acc, exact=val)

    # 2. uniform(-1,1) GEMV inputs, weight stored [N,K]
    K, N = 384, 128
    x = (rng.random((1, K)) * 2 - 1).astype(np.float16)
    Wt = (rng.random((N, K)) * 2 - 1).astype(np.float16)
    exp, val = exact_gemm(x.view(np.uint16), np.ascontiguousarray(Wt.T).view(np.uint16))
    np.savez_compressed(HERE / "gemv_uniform.npz", x=x.view(np.uint16), W_nk=Wt.view(np.uint16),
                        expected=exp, exact=val)

    # 3. dyadic inputs (multiples of 1/64, |v| < 32): every fp64 partial sum is exact
    M, K, N = 2, 512, 128
    A = (rng.integers(-2047, 2048, (M, K)) / 64.0).astype(np.float16)
    W = (rng.integers(-2047, 2048, (K, N)) / 64.0).astype(np.float16)
    exp, val = exact_gemm(A.view(np.uint16), W.view(np.uint16))
    np.savez_compressed(HERE / "gemm_dyadic.npz", A=A.view(np.uint16), W_kn=W.view(np.uint16),
                        expected=exp, exact=val)

    # 4. fp16 subnormal weights and mixed magnitudes
    M, K, N = 1, 128, 128
    A = (rng.standard_normal((M, K)) * 4).astype(np.float16)
    Wb = rng.integers(0, 0x0400, (K, N)).astype(np.uint16)  # subnormals
    Wb[::3] = (rng.standard_normal((len(Wb[::3]), N)) * 1e-3).astype(np.float16).view(np.uint16)
    Wb |= (rng.integers(0, 2, (K, N)).astype(np.uint16) << 15)
    exp, val = exact_gemm(A.view(np.uint16), Wb)
    np.savez_compressed(HERE / "gemm_subnormal.npz", A=A.view(np.uint16), W_kn=Wb, expected=exp, exact=val)

    # 5. int8 GEMV: exact integer dot, and the W8A16 sum with fp16 activations
    K, N = 256, 128
    Wq = rng.integers(-128, 128, (N, K)).astype(np.int8)
    xq = rng.integers(-128, 128, (2, K)).astype(np.int8)
    acc = np.array([[sum(int(xq[m, k]) * int(Wq[n, k]) for k in range(K)) for n in range(N)]
                    for m in range(2)], dtype=np.int64)
    x = rng.standard_normal((1, K)).astype(np.float16)
    xi = [f16_to_int24(int(v)) for v in x.view(np.uint16)[0]]
    y_bits = np.zeros((1, N), np.uint16)
    y_val = np.zeros((1, N), np.float64)
    for n in range(N):
        s = sum(xi[k] * int(Wq[n, k]) for k in range(K))  # units of 2^-24
        y_bits[0, n] = round_f16(s, 24)
        y_val[0, n] = s / float(1 << 24)
    np.savez_compressed(HERE / "gemv_int8.npz", Wq=Wq, xq=xq, acc=acc.astype(np.int32), x=x.view(np.uint16),
                        y_expected=y_bits, y_exact=y_val)
    # 6. int4 GEMV: two unsigned nibbles per byte, even element in the low nibble, zero point 8
    K, N = 256, 128
    Wq4 = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    x = rng.standard_normal((2, K)).astype(np.float16)
    y_bits = np.zeros((2, N), np.uint16)
    y_val = np.zeros((2, N), np.float64)
    for m in range(2):
        xi = [f16_to_int24(int(v)) for v in x.view(np.uint16)[m]]
        for n in range(N):
            s = 0
            for b in range(K // 2):
                byte = int(Wq4[n, b])
                s += xi[2 * b] * ((byte & 15) - 8) + xi[2 * b + 1] * ((byte >> 4) - 8)  # units of 2^-24
            y_bits[m, n] = round_f16(s, 24)
            y_val[m, n] = s / float(1 << 24)
    np.savez_compressed(HERE / "gemv_int4.npz", Wq4=Wq4, x=x.view(np.uint16), y_expected=y_bits, y_exact=y_val)
    print("wrote", sorted(p.name for p in HERE.glob("*.npz")))


if __name__ == "__main__":
    main()
