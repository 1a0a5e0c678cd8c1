"""The library's own plan at real sizes, over a grid of shapes that reaches every branch of the
planner (tile widths 16 / 32 / 48 / 64 and ragged, 128- and 256-byte bands, splits of narrow
outputs, both v_dot2 kernels, the 4x4x4 kernel's zone) and of the int8 launcher.

Weights are generated on the device.  Every output is held to the tolerance against an fp32
product computed on the device (a size-independent check of all M x N values), and a spread of
output columns -- both ends of N plus a seeded sample -- against the oracle, for which the matching
weight rows are copied to the host.
"""
import numpy as np
import pytest
import torch

import oracle
from fastgate_amd import capi
from helpers import ATOL, RTOL, assert_close_f16

pytestmark = pytest.mark.gpu

NS = (1024, 2048, 3072, 5120, 6144, 7168, 8192, 9216, 11008, 12288, 14336, 16384)
KS = (2048, 4096, 6144, 8192, 11008)
MS = (1, 3, 6, 9, 13, 16, 24)


@pytest.fixture(scope="module")
def sg():
    import fastgate_amd

    return fastgate_amd.speedgate


def _cols(N, seed):
    rng = np.random.default_rng(seed)
    return np.unique(np.concatenate([np.arange(8), np.arange(N - 8, N), rng.integers(0, N, 32)]))


def _within_tolerance(C, ref32, what):
    err = (C.float() - ref32).abs()
    tol = ATOL + RTOL * ref32.abs()
    assert torch.isfinite(C).all(), what
    worst = (err - tol).max().item()
    assert worst <= 0.0, "%s: %.4g beyond the tolerance" % (what, worst)


@pytest.mark.parametrize("K", KS)
def test_fp16_library_plans_over_the_shape_grid(device, sg, K):
    gd = torch.Generator(device=device)
    seen = set()
    for N in NS:
        gd.manual_seed(7000 + N + K)
        Wt = (torch.randn((N, K), device=device, generator=gd) * 0.02).half()
        Wkn = Wt.t().contiguous()
        W32 = Wt.float()
        cols = _cols(N, N + K)
        Wsub = np.ascontiguousarray(Wt[torch.from_numpy(cols).to(device)].cpu().numpy())
        for M in MS:
            A = torch.randn((M, K), device=device, generator=gd).half()
            ref32 = A.float() @ W32.t()
            ref, _ = oracle.gemm_f16(A.cpu().numpy(), Wsub, oracle.W_NK)
            for layout, op, W in ((capi.FG_W_NK, sg.edgemm_m8n128k64x4_bt, Wt),
                                  (capi.FG_W_KN, sg.edgemm_m8n128k64x4, Wkn)):
                p = capi.plan(M, N, K, layout, 0)
                seen.add((p.kernel, p.tile_n if layout == capi.FG_W_NK else 0, p.band, p.splitk > 1))
                what = "%s M=%d N=%d K=%d %s" % ("[N,K]" if layout == capi.FG_W_NK else "[K,N]", M, N, K,
                                               p.as_dict())
                C = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
                op(A, W, C)
                _within_tolerance(C, ref32, what)
                assert_close_f16(C[:, torch.from_numpy(cols).to(device)].cpu().numpy(), ref, what)
        del Wt, Wkn, W32
    # the grid is only worth its time if it reaches the planner's branches
    kernels = {k for k, _, _, _ in seen}
    assert {capi.FG_KERNEL_NK_DOT2, capi.FG_KERNEL_NK_MFMA_R, capi.FG_KERNEL_KN_DOT2,
            capi.FG_KERNEL_KN_MFMA} <= kernels
    assert len({t for k, t, _, _ in seen if k == capi.FG_KERNEL_NK_MFMA_R}) >= 4


@pytest.mark.parametrize("K", (2048, 4096, 8192, 14336))
def test_int8_launcher_over_the_shape_grid(device, sg, K):
    gd = torch.Generator(device=device)
    for N in (1024, 2048, 4096, 5120, 6144, 8192, 11008, 14336, 16384):
        gd.manual_seed(7100 + N + K)
        Wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=device, generator=gd)
        scale = (torch.rand(N, device=device, generator=gd) * 0.0009 + 0.0001).half()
        cols = _cols(N, N + K + 1)
        ct = torch.from_numpy(cols).to(device)
        Wsub = np.ascontiguousarray(Wq[ct].cpu().numpy())
        ssub = scale[ct].cpu().numpy()
        W32 = Wq.float()
        for M in (1, 2, 4, 7, 8, 12, 13, 16):
            x = torch.randn((M, K), device=device, generator=gd).half()
            y = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
            sg.fastgemv_int8(Wq, x, y, scale=scale, zero_point=2.0)
            what = "W8A16 M=%d N=%d K=%d" % (M, N, K)
            x32 = x.float()
            ref32 = (x32 @ W32.t() - 2.0 * x32.sum(dim=1, keepdim=True)) * scale.float()
            _within_tolerance(y, ref32, what)
            ref, _ = oracle.gemv_w8a16(Wsub, x.cpu().numpy(), ssub, 1.0, 2.0)
            assert_close_f16(y[:, ct].cpu().numpy(), ref.reshape(M, -1), what)
        del Wq, W32
