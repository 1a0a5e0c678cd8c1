"""The GPU path against the committed golden vectors (tests/golden/*.npz: expected fp16 bits from
exact integer arithmetic, no oracle code involved), through the pybind operators."""
from pathlib import Path

import numpy as np
import pytest
import torch

from helpers import assert_close_f16

pytestmark = pytest.mark.gpu

GOLD = Path(__file__).resolve().parent / "golden"


@pytest.fixture(scope="module")
def sg():
    import fastgate_amd

    return fastgate_amd.speedgate


def _h(bits):
    return torch.from_numpy(bits.view(np.float16).copy())


def _ulps(a_bits, b_bits):
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


@pytest.mark.parametrize("name", ["gemm_normal", "gemm_dyadic", "gemm_subnormal"])
def test_gemm_fixtures_both_layouts(device, sg, name):
    z = np.load(GOLD / (name + ".npz"))
    A, Wkn = _h(z["A"]).to(device), _h(z["W_kn"]).to(device)
    want = z["expected"]
    M, N = want.shape
    C = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
    sg.edgemm_m8n128k64x4(A, Wkn, C)
    got = C.cpu().numpy()
    # fp32 accumulation against the exactly rounded value: at most one fp16 ulp apart
    assert _ulps(got.view(np.uint16), want).max() <= 1
    C.fill_(float("nan"))
    sg.edgemm_m8n128k64x4_bt(A, Wkn.t().contiguous(), C)
    assert _ulps(C.cpu().numpy().view(np.uint16), want).max() <= 1
    if name == "gemm_dyadic":   # every partial sum is exact in fp32: bit for bit
        assert (got.view(np.uint16) == want).all()
    if "expected_accumulate" in z.files:
        C0 = _h(z["C0"]).to(device)
        Ca = C0.clone()
        sg.flat_gemm_m8n256k64x8(A, Wkn, Ca, 0)          # C += A·W
        assert _ulps(Ca.cpu().numpy().view(np.uint16), z["expected_accumulate"]).max() <= 1
        Ca = C0.clone()
        sg.gemm_m8n32k256x8_bt(A, Wkn.t().contiguous(), Ca)
        assert _ulps(Ca.cpu().numpy().view(np.uint16), z["expected_accumulate"]).max() <= 1


def test_gemv_fixture_weight_first(device, sg):
    z = np.load(GOLD / "gemv_uniform.npz")
    W, x = _h(z["W_nk"]).to(device), _h(z["x"]).to(device)
    y = torch.full((W.shape[0],), float("nan"), dtype=torch.half, device=device)
    for op in (sg.fastgemv, sg.fastgemv_tuned, sg.fastgemv_extend, sg.fastgemm):
        y.fill_(float("nan"))
        op(W, x, y)
        assert _ulps(y.cpu().numpy().view(np.uint16), z["expected"][0]).max() <= 1


def test_int8_fixture(device, sg):
    z = np.load(GOLD / "gemv_int8.npz")
    Wq = torch.from_numpy(z["Wq"]).to(device)
    xq = torch.from_numpy(z["xq"]).to(device)
    acc = torch.full(tuple(z["acc"].shape), -1, dtype=torch.int32, device=device)
    sg.gemv_i8i8_i32(Wq, xq, acc)
    assert (acc.cpu().numpy() == z["acc"]).all()
    x = _h(z["x"]).to(device)
    y = torch.full((Wq.shape[0],), float("nan"), dtype=torch.half, device=device)
    sg.fastgemv_int8(Wq, x, y)
    assert _ulps(y.cpu().numpy().view(np.uint16), z["y_expected"][0]).max() <= 1
    assert_close_f16(y.cpu().numpy(), z["y_expected"][0].view(np.float16), "golden int8")
