"""GPU parity of the int8-weight GEMV kernels: the W8A16 path against the fp32 oracle within
tolerance, the integer stage bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from fastgate_amd import capi
from helpers import assert_close_f16, gen, normal, ptr, stream_ptr

pytestmark = pytest.mark.gpu


def _w8a16(Wq, x, scale, scalar_scale, zp, device):
    L = capi.lib()
    N, K = Wq.shape
    M = x.shape[0]
    y = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
    Wd, xd = Wq.to(device), x.to(device)
    sd = None if scale is None else scale.to(device)
    capi.check(L.fg_gemv_w8a16(ptr(Wd), ptr(xd), ptr(sd), scalar_scale, zp, ptr(y), M, N, K,
                               stream_ptr()), "fg_gemv_w8a16")
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 9, 13, 16])
@pytest.mark.parametrize("N,K", [(128, 128), (256, 1152), (1024, 4096), (4096, 1024), (3072, 640)])
def test_w8a16_matches_oracle(device, M, N, K):
    g = gen(4000 + M + N)
    x = normal((M, K), g)
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    ref, _ = oracle.gemv_w8a16(Wq.numpy(), x.numpy(), scale.numpy(), 1.0, 0.0)
    assert_close_f16(_w8a16(Wq, x, scale, 1.0, 0.0, device), ref, "per-channel scale")
    # the reference's effective configuration: scalar scale 1, zero point 0, no vector
    ref, _ = oracle.gemv_w8a16(Wq.numpy(), (x * 0.01).half().numpy(), None, 1.0, 0.0)
    assert_close_f16(_w8a16(Wq, (x * 0.01).half(), None, 1.0, 0.0, device), ref, "reference default")
    # scalar scale and zero point (kernel formula hk/fastgemv.cuh:344-363)
    ref, _ = oracle.gemv_w8a16(Wq.numpy(), x.numpy(), scale.numpy(), 0.5, 3.0)
    assert_close_f16(_w8a16(Wq, x, scale, 0.5, 3.0, device), ref, "scale 0.5 zp 3")


@pytest.mark.parametrize("M", [3, 4, 5, 7, 8, 9, 12, 16])
@pytest.mark.parametrize("N,K", [(16384, 128), (16384, 384), (16384, 1152), (32768, 384), (14336, 640), (5120, 384)])
def test_w8a16_wide_tiles_for_wide_outputs(device, M, N, K):
    # N / 32 a multiple of 512 or 448..512 (13..16 rows: from 160): 32-column tiles on 128-byte
    # bands, 4-, 8- or 16-row activation
    # strips; exact small integers first (any LDS layout mistake changes the bits), then random data
    g = gen(4100 + M + N + K)
    xi = torch.randint(-3, 4, (M, K), generator=g).half()
    Wsmall = torch.randint(-8, 9, (N, K), generator=g, dtype=torch.int8)
    ref, _ = oracle.gemv_w8a16(Wsmall.numpy(), xi.numpy(), None, 1.0, 0.0)
    got = _w8a16(Wsmall, xi, None, 1.0, 0.0, device)
    exact = np.abs(ref.astype(np.float32)) <= 2048
    assert (got[exact] == ref[exact]).all() and exact.mean() > 0.9
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    x = normal((M, K), g)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    ref, _ = oracle.gemv_w8a16(Wq.numpy(), x.numpy(), scale.numpy(), 0.5, 3.0)
    assert_close_f16(_w8a16(Wq, x, scale, 0.5, 3.0, device), ref, "scale 0.5 zp 3")


@pytest.mark.parametrize("M,K", [(4, 16384), (8, 16384), (13, 16384), (16, 4096), (6, 24576)])
def test_w8a16_wide_tiles_with_one_workgroup_per_cu(device, M, K):
    # N = 8192: 256 tiles of 32 columns, taken for long rows or 15..16 activation rows; the oracle
    # checks three windows of output channels, exact integers first
    N = 8192
    g = gen(4190 + M + K)
    xi = torch.randint(-1, 2, (M, K), generator=g).half()
    Wsmall = torch.randint(-2, 3, (N, K), generator=g, dtype=torch.int8)
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    x = normal((M, K), g)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    got_small = _w8a16(Wsmall, xi, None, 1.0, 0.0, device)
    got = _w8a16(Wq, x, scale, 0.5, 3.0, device)
    for lo in (0, 4080, N - 96):
        ref, _ = oracle.gemv_w8a16(Wsmall[lo:lo + 96].numpy(), xi.numpy(), None, 1.0, 0.0)
        assert np.abs(ref.astype(np.float32)).max() <= 2048
        assert (got_small[:, lo:lo + 96] == ref).all()
        ref, _ = oracle.gemv_w8a16(Wq[lo:lo + 96].numpy(), x.numpy(), scale[lo:lo + 96].numpy(), 0.5, 3.0)
        assert_close_f16(got[:, lo:lo + 96], ref, "rows %d.." % lo)


@pytest.mark.parametrize("M", [5, 8])
def test_w8a16_long_rows_of_narrow_outputs_use_256_byte_bands(device, M):
    # N <= 4096 and K >= 14336: 256-byte bands (8-row strips); K = 113 bands of 128 leaves the
    # last 256-byte band half empty.  Exact integers first, then random data
    N, K = 2560, 14336 + 128
    g = gen(4170 + M)
    xi = torch.randint(-1, 2, (M, K), generator=g).half()
    Wsmall = torch.randint(-2, 3, (N, K), generator=g, dtype=torch.int8)
    ref, _ = oracle.gemv_w8a16(Wsmall.numpy(), xi.numpy(), None, 1.0, 0.0)
    got = _w8a16(Wsmall, xi, None, 1.0, 0.0, device)
    assert np.abs(ref.astype(np.float32)).max() <= 2048
    assert (got == ref).all()
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    x = normal((M, K), g)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    ref, _ = oracle.gemv_w8a16(Wq.numpy(), x.numpy(), scale.numpy(), 0.5, 3.0)
    assert_close_f16(_w8a16(Wq, x, scale, 0.5, 3.0, device), ref, "scale 0.5 zp 3")


@pytest.mark.parametrize("M", [9, 11, 16])
@pytest.mark.parametrize("N,K", [(1024, 128), (2048, 640), (8192, 1152)])
def test_w8a16_16_row_strip_is_exact_on_small_integers(device, M, N, K):
    # 9..16 activation rows: 16-row strip, 16-column tiles.  Integer data whose sums fp16 holds
    # exactly: a wrong row, band or byte in the staged strips changes the bits
    g = gen(4150 + M + N + K)
    xi = torch.randint(-3, 4, (M, K), generator=g).half()
    Wsmall = torch.randint(-8, 9, (N, K), generator=g, dtype=torch.int8)
    ref, _ = oracle.gemv_w8a16(Wsmall.numpy(), xi.numpy(), None, 1.0, 0.0)
    got = _w8a16(Wsmall, xi, None, 1.0, 0.0, device)
    exact = np.abs(ref.astype(np.float32)) <= 2048
    assert (got[exact] == ref[exact]).all() and exact.mean() > 0.9
    # each row alone gives the same bits as within the batch
    one = _w8a16(Wsmall, xi[M - 1:M].contiguous(), None, 1.0, 0.0, device)
    assert (one[0] == got[M - 1]).all()


@pytest.mark.parametrize("M", [2, 3])
def test_w8a16_large_weights_with_a_ragged_last_band(device, M):
    # K = 65 bands of 128: the last 256-byte band of a row is half empty; the oracle checks
    # three windows of output channels
    N, K = 16384, 8192 + 128
    g = gen(880 + M)
    x = normal((M, K), g, 1.0)
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    got = _w8a16(Wq, x, scale, 1.0, 2.0, device)
    for lo in (0, 8000, N - 144):
        ref, _ = oracle.gemv_w8a16(Wq[lo:lo + 144].numpy(), x.numpy(), scale[lo:lo + 144].numpy(), 1.0, 2.0)
        assert_close_f16(got[:, lo:lo + 144], ref, "rows %d.." % lo)


def test_w8a16_every_int8_value_is_exact(device):
    # x = e_k picks single weights: the result must be the int8 value itself, all 256 of them.
    N, K = 256, 128
    Wq = torch.arange(-128, 128, dtype=torch.int16).to(torch.int8).reshape(N, 1).repeat(1, K).contiguous()
    for k in (0, 1, 2, 3, 17, 127):
        x = torch.zeros((1, K), dtype=torch.half)
        x[0, k] = 1.0
        got = _w8a16(Wq, x, None, 1.0, 0.0, device)
        assert (got[0] == np.arange(-128, 128, dtype=np.float16)).all()


def test_w8a16_byte_order_within_chunk(device):
    # weights 1..16 along k against x = e_k: catches a swapped byte / pair mapping
    N, K = 128, 256
    Wq = (torch.arange(K) % 16 + 1).to(torch.int8).repeat(N, 1).contiguous()
    for k in range(0, 48):
        x = torch.zeros((1, K), dtype=torch.half)
        x[0, k] = 2.0
        got = _w8a16(Wq, x, None, 1.0, 0.0, device)
        assert (got == 2.0 * (k % 16 + 1)).all(), k


def _i8i8(Wq, xq, device):
    L = capi.lib()
    N, K = Wq.shape
    M = xq.shape[0]
    acc = torch.full((M, N), -7, dtype=torch.int32, device=device)
    Wd, xd = Wq.to(device), xq.to(device)
    capi.check(L.fg_gemv_i8i8_i32(ptr(Wd), ptr(xd), ptr(acc), M, N, K, stream_ptr()),
               "fg_gemv_i8i8_i32")
    torch.cuda.synchronize()
    return acc.cpu().numpy()


@pytest.mark.parametrize("M", [1, 2, 4, 7, 8])
@pytest.mark.parametrize("N,K", [(128, 128), (384, 2176), (2048, 8192)])
def test_integer_stage_bit_exact(device, M, N, K):
    g = gen(5000 + M + K)
    Wq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    xq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    ref = oracle.gemv_i8i8_i32(Wq.numpy(), xq.numpy())
    assert (ref == (xq.numpy().astype(np.int64) @ Wq.numpy().astype(np.int64).T)).all()
    got = _i8i8(Wq, xq, device)
    assert (got == ref).all()


def test_integer_stage_extremes(device):
    # all -128 x -128 at K = 8192: 2^14 * 2^13 = 2^27, the largest magnitude reachable
    N, K = 128, 8192
    Wq = torch.full((N, K), -128, dtype=torch.int8)
    xq = torch.full((1, K), -128, dtype=torch.int8)
    assert (_i8i8(Wq, xq, device) == 128 * 128 * K).all()
    xq = torch.full((1, K), 127, dtype=torch.int8)
    assert (_i8i8(Wq, xq, device) == -128 * 127 * K).all()


def test_w8a8_dequant_epilogue(device):
    L = capi.lib()
    g = gen(6001)
    M, N, K = 2, 1024, 2048
    x = normal((M, K), g)
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    s_x = float(x.abs().max()) / 127.0
    xq = torch.clamp(torch.round(x.float() / s_x), -127, 127).to(torch.int8)
    acc_ref = oracle.gemv_i8i8_i32(Wq.numpy(), xq.numpy())
    y_ref = oracle.dequant_i32_f16(acc_ref, scale.numpy(), s_x)
    acc = torch.from_numpy(_i8i8(Wq, xq, device)).to(device)
    y = torch.empty((M, N), dtype=torch.half, device=device)
    sd = scale.to(device)
    capi.check(L.fg_dequant_i32_f16(ptr(acc), ptr(sd), s_x, ptr(y), M, N, stream_ptr()), "dequant")
    torch.cuda.synchronize()
    # same integer input, same two fp32 multiplications: identical bits
    assert (y.cpu().numpy().view(np.uint16) == y_ref.view(np.uint16)).all()


def test_int8_error_codes(device):
    L = capi.lib()
    W = torch.zeros((128, 128), dtype=torch.int8, device=device)
    x = torch.zeros((1, 128), dtype=torch.half, device=device)
    y = torch.zeros((1, 128), dtype=torch.half, device=device)
    assert L.fg_gemv_w8a16(ptr(W), ptr(x), None, 1.0, 0.0, ptr(y), 17, 128, 128, stream_ptr()) == capi.FG_ERR_INVALID_ARG
    assert L.fg_gemv_w8a16(ptr(W), ptr(x), None, 1.0, 0.0, ptr(y), 1, 100, 128, stream_ptr()) == capi.FG_ERR_ALIGN128
    assert L.fg_gemv_w8a16(None, ptr(x), None, 1.0, 0.0, ptr(y), 1, 128, 128, stream_ptr()) == capi.FG_ERR_INVALID_ARG


# ---------------------------------------------------------------------------------------
# int4 weights (two unsigned nibbles per byte, even element in the low nibble)
# ---------------------------------------------------------------------------------------
def _w4a16(Wq4, x, scale, scalar_scale, zp, device):
    L = capi.lib()
    M = x.shape[0]
    N, K = Wq4.shape[0], Wq4.shape[1] * 2
    y = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
    Wd, xd = Wq4.to(device), x.to(device)
    sd = None if scale is None else scale.to(device)
    capi.check(L.fg_gemv_w4a16(ptr(Wd), ptr(xd), ptr(sd), scalar_scale, zp, ptr(y), M, N, K,
                               stream_ptr()), "fg_gemv_w4a16")
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("M", [1, 2, 3, 4])
@pytest.mark.parametrize("N,K", [(128, 128), (256, 1152), (1024, 4096), (512, 8192 + 384)])
def test_w4a16_matches_oracle(device, M, N, K):
    g = gen(900 + M + N + K)
    x = normal((M, K), g, 1.0)
    Wq4 = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    ref, _ = oracle.gemv_w4a16(Wq4.numpy(), x.numpy(), scale.numpy(), 1.0, 8.0)
    assert_close_f16(_w4a16(Wq4, x, scale, 1.0, 8.0, device), ref, "per-channel scale, zero point 8")
    ref, _ = oracle.gemv_w4a16(Wq4.numpy(), (x * 0.01).half().numpy(), None, 1.0, 0.0)
    assert_close_f16(_w4a16(Wq4, (x * 0.01).half(), None, 1.0, 0.0, device), ref, "no scale, no zero point")
    ref, _ = oracle.gemv_w4a16(Wq4.numpy(), x.numpy(), scale.numpy(), 0.5, 7.5)
    assert_close_f16(_w4a16(Wq4, x, scale, 0.5, 7.5, device), ref, "scale 0.5 zp 7.5")


@pytest.mark.parametrize("M", [1, 2, 4])
def test_w4a16_every_nibble_in_every_position_is_exact(device, M):
    # x = e_k picks single weights: the result must be the nibble itself, for all 32 positions of
    # a 16-byte load and all 16 values (M = 1 runs the dot2 kernel, M >= 2 the row-load kernels)
    N, K = 128, 128
    Wq4 = torch.zeros((N, K // 2), dtype=torch.uint8)
    for n in range(N):
        for b in range(K // 2):
            lo, hi = (n + b) % 16, (n + 3 * b + 5) % 16
            Wq4[n, b] = lo | (hi << 4)
    want = np.empty((N, K), np.float32)
    want[:, 0::2] = (Wq4 & 0x0F).numpy()
    want[:, 1::2] = (Wq4 >> 4).numpy()
    for k in range(0, K, M):
        x = torch.zeros((M, K), dtype=torch.half)
        for m in range(M):
            x[m, k + m] = 1.0
        got = _w4a16(Wq4, x, None, 1.0, 0.0, device)
        for m in range(M):
            assert (got[m] == want[:, k + m]).all(), (k, m)


def test_w4a16_row_load_band_positions_are_exact(device):
    # a 512-element band and its partial successor: single weights picked out at positions spread
    # over both, with a zero point, must come back exactly
    g = gen(955)
    N, K = 128, 512 + 256
    Wq4 = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
    want = np.empty((N, K), np.float32)
    want[:, 0::2] = (Wq4 & 0x0F).numpy()
    want[:, 1::2] = (Wq4 >> 4).numpy()
    for k in range(0, K - 3, 37):
        x = torch.zeros((3, K), dtype=torch.half)
        for m in range(3):
            x[m, k + m] = 1.0
        got = _w4a16(Wq4, x, None, 1.0, 8.0, device)
        for m in range(3):
            assert (got[m] == want[:, k + m] - 8.0).all(), (k, m)


def test_w4a16_small_integers_are_exact(device):
    g = gen(950)
    N, K = 256, 2048
    Wq4 = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
    x = torch.randint(-4, 5, (3, K), generator=g).half()
    ref, ref32 = oracle.gemv_w4a16(Wq4.numpy(), x.numpy(), None, 1.0, 8.0)
    got = _w4a16(Wq4, x, None, 1.0, 8.0, device)
    assert (got == ref).all()


def test_w4a16_pybind_and_errors(device):
    import fastgate_amd
    sg = fastgate_amd.speedgate
    g = gen(960)
    N, K = 256, 512
    Wq4 = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
    x = normal((2, K), g, 1.0)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    y = torch.empty((2, N), dtype=torch.half, device=device)
    sg.fastgemv_int4(Wq4.to(device), x.to(device), y, scale=scale.to(device), zero_point=8.0)
    ref, _ = oracle.gemv_w4a16(Wq4.numpy(), x.numpy(), scale.numpy(), 1.0, 8.0)
    assert_close_f16(y.cpu().numpy(), ref, "fastgemv_int4")
    with pytest.raises(ValueError):
        sg.fastgemv_int4(Wq4[:100].contiguous().to(device), x.to(device), y)
    with pytest.raises(RuntimeError):
        sg.fastgemv_int4(Wq4.to(device).to(torch.int8), x.to(device), y)
    L = capi.lib()
    W = Wq4.to(device)
    xd = x.to(device)
    assert L.fg_gemv_w4a16(ptr(W), ptr(xd), None, 1.0, 0.0, ptr(y), 5, N, K, stream_ptr()) == capi.FG_ERR_INVALID_ARG
    assert L.fg_gemv_w4a16(ptr(W), ptr(xd), None, 1.0, 0.0, ptr(y), 1, 100, K, stream_ptr()) == capi.FG_ERR_ALIGN128


def test_w4a16_golden_vectors(device):
    # exact-integer expected values (tests/golden/make_golden.py), two rows at once and one by one
    from pathlib import Path
    z = np.load(Path(__file__).resolve().parent / "golden" / "gemv_int4.npz")
    Wq4 = torch.from_numpy(z["Wq4"])
    x = torch.from_numpy(z["x"].view(np.float16).copy())
    want = z["y_expected"].view(np.float16)
    assert_close_f16(_w4a16(Wq4, x, None, 1.0, 8.0, device), want, "golden int4, M=2")
    for m in range(2):
        assert_close_f16(_w4a16(Wq4, x[m:m + 1].contiguous(), None, 1.0, 8.0, device), want[m:m + 1], "golden int4 row %d" % m)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("N,K", [(128, 128), (128, 1152), (256, 2176), (128, 4224), (128, 9344)])
def test_one_row_kernels_pick_every_position_exactly(device, bits, N, K):
    """One activation row, x = 2^e at a single k: the output column is that weight times 2^e,
    exactly, for positions across every unit, chunk and wave of the row (a full chunk is 1024 k
    of int8 or 2048 k of int4; these K end inside a chunk) and for activations down in the fp16
    subnormal range, where the weights themselves travel as subnormals."""
    g = gen(6100 + bits + K)
    if bits == 8:
        W = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
        want = W.numpy().astype(np.float32)
        run = _w8a16
    else:
        W = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
        want = np.empty((N, K), np.float32)
        want[:, 0::2] = (W & 0x0F).numpy()
        want[:, 1::2] = (W >> 4).numpy()
        run = _w4a16
    ks = sorted(set(list(range(0, 40)) + list(range(K - 40, K)) + list(range(5, K, 263)) +
                    [k for c in range(512, K, 512) for k in (c - 1, c)]))
    for i, k in enumerate(ks):
        e = (0, -3, -14, -17, -24)[i % 5]            # 2^-17 and 2^-24 are fp16 subnormals
        x = torch.zeros((1, K), dtype=torch.half)
        x[0, k] = 2.0 ** e
        got = run(W, x, None, 1.0, 0.0, device).astype(np.float64)
        expect = (want[:, k].astype(np.float64) * 2.0 ** e).astype(np.float16).astype(np.float64)
        assert (got[0] == expect).all(), (k, e)


@pytest.mark.parametrize("bits", [4, 8])
def test_one_row_kernels_small_integers_and_zero_point_are_exact(device, bits):
    g = gen(6200 + bits)
    for (N, K) in ((256, 2048), (128, 3200), (512, 8192), (128, 20480)):
        x = torch.randint(-3, 4, (1, K), generator=g).half()
        if bits == 8:
            W = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
            ref, _ = oracle.gemv_w8a16(W.numpy(), x.numpy(), None, 1.0, 3.0)
            got = _w8a16(W, x, None, 1.0, 3.0, device)
        else:
            W = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
            ref, _ = oracle.gemv_w4a16(W.numpy(), x.numpy(), None, 1.0, 8.0)
            got = _w4a16(W, x, None, 1.0, 8.0, device)
        # every fp32 sum on the way is an integer below 2^24: the one rounding to fp16 decides
        assert (got.view(np.uint16) == ref.view(np.uint16)).all(), (N, K)


@pytest.mark.parametrize("bits,M,N", [(8, 1, 1024), (8, 2, 1024), (8, 4, 1024), (8, 4, 4096), (8, 8, 4096),
                                      (8, 16, 2048), (8, 16, 16384), (4, 1, 1024), (4, 2, 512), (4, 4, 512)])
@pytest.mark.parametrize("zp", [0.0, 3.0])
def test_infinite_and_nan_activations_keep_the_class_of_element_by_element_sums(device, bits, M, N, zp):
    # hk/fastgemv.cuh:344-363 adds x (float(w) - zp) element by element: +inf against weights above the
    # zero point gives +inf, below it -inf, on it NaN; infinities of both signs or a NaN give NaN.
    # The kernels take the zero point (and int8's + 128) out as one term with Σx, which alone would
    # make every such output NaN; rows with finite activations must not notice their neighbours.
    K = 1152
    g = gen(6300 + bits + M + N)
    x = normal((M, K), g)
    k0, k1 = 5, 700
    x[0, k0] = float("inf")
    if M > 1:
        x[1, k1] = float("nan")
    if M > 2:
        x[2, k0], x[2, k1] = float("inf"), float("-inf")
    if M > 3:
        x[3, k1] = float("-inf")
    third = N // 3
    if bits == 8:
        W = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
        W[:third, k0] = int(zp)        # on the zero point: NaN
        W[third:2 * third, k0] = 100   # above: the sign of the infinity
        W[2 * third:, k0] = -100       # below: the other sign
        W[::2, k1] = 50
        W[1::2, k1] = -50
        ref, _ = oracle.gemv_w8a16(W.numpy(), x.numpy(), None, 1.0, zp)
        got = _w8a16(W, x, None, 1.0, zp, device)
    else:
        W = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
        lo = lambda col, v: (col & 0xF0) | v      # k0 is odd: the high nibble; k1 even: the low one
        W[:third, k0 // 2] = (W[:third, k0 // 2] & 0x0F) | (int(zp) << 4)
        W[third:2 * third, k0 // 2] = (W[third:2 * third, k0 // 2] & 0x0F) | (12 << 4)
        W[2 * third:, k0 // 2] = (W[2 * third:, k0 // 2] & 0x0F) | (1 << 4)
        W[::2, k1 // 2] = lo(W[::2, k1 // 2], 9)
        W[1::2, k1 // 2] = lo(W[1::2, k1 // 2], 2)
        ref, _ = oracle.gemv_w4a16(W.numpy(), x.numpy(), None, 1.0, zp)
        got = _w4a16(W, x, None, 1.0, zp, device)
    assert np.isnan(ref[0, :third]).all() and np.isinf(ref[0, third:]).all()  # the case is what it claims
    assert (np.isnan(got) == np.isnan(ref)).all()
    inf = np.isinf(ref)
    assert (np.isinf(got) == inf).all() and (got[inf] == ref[inf]).all()
    broken = min(M, 4)
    assert np.isfinite(ref[broken:]).all()
    if M > broken:
        assert_close_f16(got[broken:], ref[broken:], "rows with finite activations")
