"""Pins the CPU oracle before anything is compared with it.

The reference keeps no golden vectors for this path and its own check is a live torch.matmul,
so the oracle is pinned by: exact-integer golden vectors (tests/golden, generated without any
oracle code), IEEE conversion tables from numpy, closed forms, brute force in float64, and
torch.matmul on the CPU.  Each check is chosen so that a dropped term, a swapped operand or a
wrong layout fails it.
"""
from pathlib import Path

import numpy as np
import pytest
import torch

import oracle

GOLD = Path(__file__).resolve().parent / "golden"


def _ulps(a_bits, b_bits):
    """Distance in fp16 ulps between two finite bit patterns (sign-magnitude -> ordered int)."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


# ---- conversions --------------------------------------------------------------------------
def test_h2f_every_code():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.h2f(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(ref)
    assert (np.isnan(got) == nan).all()
    assert (got[~nan].view(np.uint32) == ref[~nan].view(np.uint32)).all()


def test_f2h_round_to_nearest_even():
    rng = np.random.default_rng(1)
    vals = [rng.standard_normal(20000).astype(np.float32) * s for s in (1e-7, 1e-4, 1.0, 300.0, 7e4)]
    # every midpoint between neighbouring halves, and its two fp32 neighbours
    h = np.arange(0, 0x7BFF, dtype=np.uint16).view(np.float16).astype(np.float64)
    hn = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = ((h + hn) / 2).astype(np.float32)
    vals += [mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)), -mid]
    vals += [np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, np.inf, -np.inf, 2.0**-24,
                       2.0**-25, 2.0**-25 * 1.0001, 2.0**-14, 5.96e-8], dtype=np.float32)]
    v = np.concatenate(vals)
    with np.errstate(over="ignore"):
        ref = v.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f2h(float(x)) for x in v], dtype=np.uint16)
    assert (got == ref).all()
    assert oracle.f2h(float("nan")) & 0x7C00 == 0x7C00 and oracle.f2h(float("nan")) & 0x3FF


def test_d2h_single_rounding():
    rng = np.random.default_rng(2)
    v = np.concatenate([rng.standard_normal(20000) * s for s in (1e-7, 1e-4, 1.0, 300.0, 7e4)])
    # a value that double rounding through fp32 gets wrong: just above a half-way point
    tricky = np.float64(1.0) + 2.0**-11 + 2.0**-40
    v = np.concatenate([v, [tricky, -tricky, 0.0, 65519.999, 65520.0, 2.0**-25, 2.0**-25 + 1e-20]])
    with np.errstate(over="ignore"):
        ref = v.astype(np.float16).view(np.uint16)
    got = np.array([oracle.d2h(float(x)) for x in v], dtype=np.uint16)
    assert (got == ref).all()
    assert oracle.d2h(float(tricky)) == np.float16(1.0 + 2.0**-10).view(np.uint16)


# ---- golden vectors (exact integer arithmetic) ---------------------------------------------
def test_golden_dyadic_fp64_twin_is_bit_exact():
    z = np.load(GOLD / "gemm_dyadic.npz")
    A, W = z["A"].view(np.float16), z["W_kn"].view(np.float16)
    got, raw = oracle.gemm_f16(A, W, oracle.W_KN, acc="f64")
    assert (raw == z["exact"]).all()          # every fp64 partial sum is exact here
    assert (got.view(np.uint16) == z["expected"]).all()
    got_nk, _ = oracle.gemm_f16(A, np.ascontiguousarray(W.T), oracle.W_NK, acc="f64")
    assert (got_nk.view(np.uint16) == z["expected"]).all()
    got32, _ = oracle.gemm_f16(A, W, oracle.W_KN)
    assert _ulps(got32.view(np.uint16), z["expected"]).max() <= 1


@pytest.mark.parametrize("name", ["gemm_normal", "gemm_subnormal"])
def test_golden_random_inputs(name):
    z = np.load(GOLD / (name + ".npz"))
    A, W = z["A"].view(np.float16), z["W_kn"].view(np.float16)
    for layout, Wl in ((oracle.W_KN, W), (oracle.W_NK, np.ascontiguousarray(W.T))):
        got64, raw64 = oracle.gemm_f16(A, Wl, layout, acc="f64")
        np.testing.assert_allclose(raw64, z["exact"], rtol=1e-13, atol=1e-15)
        assert (got64.view(np.uint16) == z["expected"]).mean() > 0.999
        assert _ulps(got64.view(np.uint16), z["expected"]).max() <= 1
        got32, raw32 = oracle.gemm_f16(A, Wl, layout)
        np.testing.assert_allclose(raw32, z["exact"], rtol=2e-5, atol=1e-6)
        assert _ulps(got32.view(np.uint16), z["expected"]).max() <= 1
        assert (got32.view(np.uint16) == z["expected"]).mean() > 0.98
    if "expected_accumulate" in z.files:
        C0 = z["C0"].view(np.float16)
        acc, _ = oracle.gemm_f16(A, W, oracle.W_KN, C=C0, accumulate=True, acc="f64")
        assert _ulps(acc.view(np.uint16), z["expected_accumulate"]).max() <= 1
        assert (acc.view(np.uint16) == z["expected_accumulate"]).mean() > 0.999
        over, _ = oracle.gemm_f16(A, W, oracle.W_KN, C=C0, accumulate=False, acc="f64")
        assert (over.view(np.uint16) == z["expected"]).mean() > 0.999


def test_golden_gemv_weight_first():
    z = np.load(GOLD / "gemv_uniform.npz")
    W, x = z["W_nk"].view(np.float16), z["x"].view(np.float16)
    y = oracle.fastgemv(W, x)                 # weight is the FIRST argument
    assert _ulps(y.view(np.uint16), z["expected"][0]).max() <= 1
    y2 = oracle.fastgemv(W, x.reshape(-1, 1))  # [K,1] spelling of the same vector
    assert (y2.view(np.uint16) == y.view(np.uint16)).all()


def test_golden_int8():
    z = np.load(GOLD / "gemv_int8.npz")
    assert (oracle.gemv_i8i8_i32(z["Wq"], z["xq"]) == z["acc"]).all()
    x = z["x"].view(np.float16)
    y, y32 = oracle.gemv_w8a16(z["Wq"], x)
    np.testing.assert_allclose(y32, z["y_exact"], rtol=2e-5, atol=1e-4)
    assert _ulps(y.view(np.uint16), z["y_expected"]).max() <= 1
    assert (oracle.fastgemv_int8(z["Wq"], x).view(np.uint16) == y.view(np.uint16).reshape(-1)).all()


def test_golden_int4():
    z = np.load(GOLD / "gemv_int4.npz")
    x = z["x"].view(np.float16)
    y, y32 = oracle.gemv_w4a16(z["Wq4"], x, None, 1.0, 8.0)
    np.testing.assert_allclose(y32, z["y_exact"], rtol=2e-5, atol=1e-4)
    assert _ulps(y.view(np.uint16), z["y_expected"]).max() <= 1


# ---- closed forms and brute force ------------------------------------------------------------
def test_ones_times_ones_is_K():
    for K in (128, 1024, 2048):
        A = np.ones((2, K), np.float16)
        for layout, W in ((oracle.W_KN, np.ones((K, 256), np.float16)), (oracle.W_NK, np.ones((256, K), np.float16))):
            assert (oracle.gemm_f16(A, W, layout)[0] == K).all()


def test_unit_vectors_select_rows_and_layouts_do_not_mix():
    rng = np.random.default_rng(3)
    K, N = 128, 256
    W = rng.standard_normal((K, N)).astype(np.float16)
    for k in (0, 5, 127):
        A = np.zeros((1, K), np.float16)
        A[0, k] = 1
        assert (oracle.gemm_f16(A, W, oracle.W_KN)[0][0].view(np.uint16) == W[k].view(np.uint16)).all()
        Wt = np.ascontiguousarray(W.T)
        assert (oracle.gemm_f16(A, Wt, oracle.W_NK)[0][0].view(np.uint16) == W[k].view(np.uint16)).all()
    # a non-square W read with the wrong layout must be rejected, not silently transposed
    with pytest.raises(ValueError):
        oracle.gemm_f16(np.zeros((1, K), np.float16), np.zeros((K, N), np.float16), oracle.W_NK)


def test_brute_force_float64_tiny():
    rng = np.random.default_rng(4)
    for M in (1, 2, 3):
        A = rng.standard_normal((M, 128)).astype(np.float16)
        W = (rng.standard_normal((128, 128)) * 0.1).astype(np.float16)
        ref = np.zeros((M, 128))
        for m in range(M):
            for n in range(128):
                s = 0.0
                for k in range(128):
                    s += float(A[m, k]) * float(W[k, n])
                ref[m, n] = s
        _, raw = oracle.gemm_f16(A, W, oracle.W_KN, acc="f64")
        np.testing.assert_allclose(raw, ref, rtol=1e-14, atol=0)
        _, raw_nk = oracle.gemm_f16(A, np.ascontiguousarray(W.T), oracle.W_NK, acc="f64")
        assert (raw_nk == raw).all()


def test_fp32_sum_order_is_k_ascending():
    # 2^12 then 4096 ones: ascending k keeps every 1 (partial sums stay below 2^24)...
    K = 4224
    A = np.ones((1, K), np.float16)
    W = np.ones((K, 128), np.float16)
    W[0, :] = 4096
    _, raw = oracle.gemm_f16(A, W, oracle.W_KN)
    assert (raw == 4096 + K - 1).all()
    # ...and with 2^24 in front every later +1 is lost, which only an ascending sum shows
    W[0, :] = 4096
    A[0, 0] = 4096                      # product 2^24
    _, raw = oracle.gemm_f16(A, W, oracle.W_KN)
    assert (raw == 2.0**24).all()
    _, raw_nk = oracle.gemm_f16(A, np.ascontiguousarray(W.T), oracle.W_NK)
    assert (raw_nk == 2.0**24).all()


@pytest.mark.parametrize("M,K,N,seed", [(1, 4096, 512, 1001), (8, 4096, 256, 1002), (16, 3072, 256, 1003)])
def test_against_torch_matmul_cpu(M, K, N, seed):
    g = torch.Generator().manual_seed(seed)
    A = torch.randn((M, K), generator=g).half()
    W = (torch.randn((K, N), generator=g) * 0.02).half()
    ref32 = A.float() @ W.float()
    out, raw = oracle.gemm_f16(A.numpy(), W.numpy(), oracle.W_KN)
    np.testing.assert_allclose(raw, ref32.numpy(), rtol=1e-4, atol=2e-5)
    ref16 = ref32.half().numpy()
    # two fp32 summation orders: one fp16 ulp apart at most, except where cancellation leaves a
    # result so small that the fp32 noise (<= 2e-5 here) spans several of its ulps
    d = np.abs(out.astype(np.float64) - ref16.astype(np.float64))
    assert ((_ulps(out.view(np.uint16), ref16.view(np.uint16)) <= 1) | (d <= 4e-5)).all()
    assert (out.view(np.uint16) == ref16.view(np.uint16)).mean() > 0.97
    out_nk, _ = oracle.gemm_f16(A.numpy(), W.t().contiguous().numpy(), oracle.W_NK)
    assert (out_nk.view(np.uint16) == out.view(np.uint16)).all()


# ---- int8 ------------------------------------------------------------------------------------
def test_w8a16_formula_scale_and_zero_point():
    rng = np.random.default_rng(5)
    N, K = 128, 256
    Wq = rng.integers(-128, 128, (N, K)).astype(np.int8)
    x = rng.standard_normal((2, K)).astype(np.float16)
    scale = (rng.random(N) * 0.009 + 0.001).astype(np.float16)
    for ss, zp in ((1.0, 0.0), (0.25, 0.0), (1.0, 3.0), (0.5, -7.5)):
        _, y32 = oracle.gemv_w8a16(Wq, x, scale, ss, zp)
        ref = (x.astype(np.float64) @ (Wq.astype(np.float64) - zp).T) * ss * scale.astype(np.float64)
        np.testing.assert_allclose(y32, ref, rtol=2e-5, atol=1e-5)
    _, y32 = oracle.gemv_w8a16(Wq, x, None, 1.0, 0.0)
    np.testing.assert_allclose(y32, x.astype(np.float64) @ Wq.astype(np.float64).T, rtol=2e-5, atol=2e-3)


def test_i8i8_brute_force_and_overflow_guard():
    rng = np.random.default_rng(6)
    Wq = rng.integers(-128, 128, (128, 384)).astype(np.int8)
    xq = rng.integers(-128, 128, (3, 384)).astype(np.int8)
    assert (oracle.gemv_i8i8_i32(Wq, xq) == xq.astype(np.int64) @ Wq.astype(np.int64).T).all()
    big = np.full((1, 1 << 18), -128, np.int8)
    with pytest.raises(OverflowError):
        oracle.gemv_i8i8_i32(big, big)


def test_dequant_formula():
    acc = np.array([[100, -200, 30000, 0]], np.int32)
    scale = np.array([0.5, 0.25, 0.001, 1.0], np.float16)
    y = oracle.dequant_i32_f16(acc, scale, 0.125)
    ref = (acc.astype(np.float32) * (np.float32(0.125) * scale.astype(np.float32))).astype(np.float16)
    assert (y.view(np.uint16) == ref.view(np.uint16)).all()


# ---- operator conventions ----------------------------------------------------------------------
def test_operator_table_protocols():
    rng = np.random.default_rng(7)
    M, K, N = 4, 128, 256
    A = rng.standard_normal((M, K)).astype(np.float16)
    W = (rng.standard_normal((K, N)) * 0.1).astype(np.float16)
    C0 = rng.standard_normal((M, N)).astype(np.float16)
    plain, _ = oracle.gemm_f16(A, W, oracle.W_KN)
    added, _ = oracle.gemm_f16(A, W, oracle.W_KN, C=C0, accumulate=True)
    assert not (plain == added).all()
    for name, (layout, protocol, has_bz) in oracle.GEMM_OPS.items():
        B = W if layout == oracle.W_KN else np.ascontiguousarray(W.T)
        out = oracle.gemm_op(name, A, B, C0, bz=2 if has_bz else None)
        want = plain if protocol == "overwrite" else added
        assert (out.view(np.uint16) == want.view(np.uint16)).all(), name
        with pytest.raises(TypeError):
            oracle.gemm_op(name, A, B, C0, bz=None if has_bz else 2)
    assert len(oracle.GEMM_OPS) == 17


def test_operator_table_rejects_unaligned():
    A = np.zeros((8, 200), np.float16)
    with pytest.raises(ValueError, match="multiple of 128"):
        oracle.gemm_op("edgemm_m8n128k64x4", A, np.zeros((200, 128), np.float16), None)
    with pytest.raises(ValueError, match="multiple of 128"):
        oracle.gemm_op("edgemm_m8n128k64x4_bt", np.zeros((8, 128), np.float16), np.zeros((100, 128), np.float16), None)


# ---------------------------------------------------------------------------------------
# int4: two unsigned nibbles per byte, even element in the low nibble (hk/utility.cuh:13-36)
# ---------------------------------------------------------------------------------------
def _unpack_u4(Wq4):
    lo = (Wq4 & 0x0F).astype(np.int64)
    hi = (Wq4 >> 4).astype(np.int64)
    out = np.empty((Wq4.shape[0], Wq4.shape[1] * 2), np.int64)
    out[:, 0::2] = lo   # getX: low nibble = first element
    out[:, 1::2] = hi   # getY: high nibble = second element
    return out


def test_w4a16_nibble_order_and_every_value():
    # x = e_k picks single weights: the result is the nibble itself; byte 0xA3 holds 3 then 10
    N, K = 16, 32
    Wq4 = np.zeros((N, K // 2), np.uint8)
    Wq4[:, 0] = 0xA3
    for n in range(N):
        Wq4[n, 5] = n | ((15 - n) << 4)
    for k, want in ((0, 3.0), (1, 10.0)):
        x = np.zeros((1, K), np.float16)
        x[0, k] = 1.0
        y, _ = oracle.gemv_w4a16(Wq4, x)
        assert (y == want).all()
    x = np.zeros((2, K), np.float16)
    x[0, 10] = 1.0
    x[1, 11] = 1.0
    y, _ = oracle.gemv_w4a16(Wq4, x)
    assert (y[0] == np.arange(N)).all() and (y[1] == 15 - np.arange(N)).all()


def test_w4a16_matches_exact_integer_arithmetic():
    # integer x, integer zero point: every product and sum is an exact integer below 2^24
    rng = np.random.default_rng(404)
    N, K = 64, 512
    Wq4 = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    xi = rng.integers(-8, 9, (3, K))
    for zp in (0, 8, 3):
        want = xi @ (_unpack_u4(Wq4) - zp).T          # int64, exact
        y, y32 = oracle.gemv_w4a16(Wq4, xi.astype(np.float16), None, 1.0, float(zp))
        assert (y32.astype(np.int64) == want).all()
        assert (y.astype(np.float64) == np.float16(want).astype(np.float64)).all()
    # power-of-two scales are exact as well
    sc = np.float16(2.0) ** rng.integers(-6, 1, N)
    y, _ = oracle.gemv_w4a16(Wq4, xi.astype(np.float16), sc.astype(np.float16), 0.5, 8.0)
    want = (xi @ (_unpack_u4(Wq4) - 8).T) * 0.5 * sc.astype(np.float64)[None, :]
    assert (y.astype(np.float64) == np.float16(want).astype(np.float64)).all()


def test_w4a16_against_float64_on_random_inputs():
    rng = np.random.default_rng(405)
    N, K = 128, 1024
    Wq4 = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    x = rng.standard_normal((2, K)).astype(np.float16)
    sc = (rng.random(N) * 0.009 + 0.001).astype(np.float16)
    _, y32 = oracle.gemv_w4a16(Wq4, x, sc, 1.0, 7.5)
    want = (x.astype(np.float64) @ (_unpack_u4(Wq4) - 7.5).T) * sc.astype(np.float64)[None, :]
    assert np.abs(y32 - want).max() <= 2e-4 * np.abs(want).max()


# ---------------------------------------------------------------------------------------
# bias + activation tail: pinned by torch's float64 routines and by closed forms
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("act", ["none", "relu", "gelu", "gelu_tanh", "silu"])
def test_bias_act_matches_torch_float64(act):
    import torch
    rng = np.random.default_rng(11)
    raw = (rng.standard_normal((5, 384)) * 3).astype(np.float32)
    raw[0, :8] = [0.0, -0.0, 1.0, -1.0, 10.0, -10.0, 30.0, -30.0]
    bias = (rng.standard_normal(384)).astype(np.float16)
    x = torch.from_numpy(raw).double() + torch.from_numpy(bias).double()[None, :]
    want = {"none": lambda t: t, "relu": torch.relu, "gelu": torch.nn.functional.gelu,
            "gelu_tanh": lambda t: torch.nn.functional.gelu(t, approximate="tanh"),
            "silu": torch.nn.functional.silu}[act](x).numpy()
    y, y32 = oracle.bias_act(raw, bias, act)
    assert np.abs(y32.astype(np.float64) - want).max() <= 2e-6 * max(1.0, np.abs(want).max())
    # the fp16 result is the correctly rounded float64 value except where fp32 noise crosses a tie;
    # in the far negative tail 1 + erf cancels in fp32, so tiny outputs are held to 1e-6 absolute
    big = np.abs(want) > 1e-3
    assert (y[big] == want.astype(np.float16)[big]).mean() > 0.995
    assert np.abs(y.astype(np.float64) - want)[~big].max(initial=0.0) <= 1e-6 + 6e-8
    assert (np.abs(y.astype(np.float64) - want) <= np.spacing(np.abs(want).astype(np.float16)) + 1e-6).all()


def test_bias_act_closed_forms():
    raw = np.array([[0.0, -5.0, 5.0, 1.0]], np.float32)
    for act in ("relu", "gelu", "gelu_tanh", "silu"):
        assert oracle.bias_act(raw, None, act)[1][0, 0] == 0.0
    assert (oracle.bias_act(raw, None, "relu")[1] == [[0.0, 0.0, 5.0, 1.0]]).all()
    # silu(1) = 1/(1+1/e), gelu(1) = Phi(1)
    assert abs(oracle.bias_act(raw, None, "silu")[1][0, 3] - 0.7310585786300049) < 1e-6
    assert abs(oracle.bias_act(raw, None, "gelu")[1][0, 3] - 0.8413447460685429) < 1e-6
    # the bias is indexed by column, not by row
    raw = np.zeros((3, 128), np.float32)
    bias = np.arange(128).astype(np.float16)
    assert (oracle.bias_act(raw, bias, "none")[0] == bias[None, :]).all()
    # gemm_bias_act = product then tail
    rng = np.random.default_rng(12)
    A = rng.standard_normal((2, 128)).astype(np.float16)
    W = (rng.standard_normal((128, 128)) * 0.1).astype(np.float16)
    _, raw = oracle.gemm_f16(A, W, oracle.W_KN)
    assert (oracle.gemm_bias_act(A, W, oracle.W_KN, bias, "relu") == oracle.bias_act(raw, bias, "relu")[0]).all()
