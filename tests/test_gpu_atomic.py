"""Split-K completion through one fixed-point atomic per output element (plan.fused = 2): every
kernel family against the oracle and against the two-pass completion, special values, the limits
of the protocol, and the workspace header going back to zero."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from fastgate_amd import capi
from helpers import assert_close_f16, gen, make_plan, normal, ptr, stream_ptr

pytestmark = pytest.mark.gpu

KN, NK = capi.FG_W_KN, capi.FG_W_NK

FAMILIES = [
    ("nk_dot2", NK, dict(kernel=capi.FG_KERNEL_NK_DOT2, tile_n=4, m_block=2, unroll=1)),
    ("nk_mfma4", NK, dict(kernel=capi.FG_KERNEL_NK_MFMA4, tile_n=16, m_block=8, unroll=1)),
    ("nk_mfma_r", NK, dict(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=16, unroll=1, waves=8)),
    ("nk_mfma_r 32 columns", NK, dict(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=32, unroll=1, waves=8, band=128)),
    ("kn_dot2", KN, dict(kernel=capi.FG_KERNEL_KN_DOT2, m_block=2, unroll=1)),
    ("kn_dot2 four rows", KN, dict(kernel=capi.FG_KERNEL_KN_DOT2, m_block=4, unroll=1)),
    ("kn_mfma", KN, dict(kernel=capi.FG_KERNEL_KN_MFMA, unroll=1)),
    ("kn_mfma eight waves", KN, dict(kernel=capi.FG_KERNEL_KN_MFMA, unroll=2, waves=8)),
]


def _ulps(a, b):
    def key(x):
        x = x.view(np.uint16).astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a) - key(b))


def _run(A, W, layout, device, plan, accumulate=False, C0=None, ws=None):
    L = capi.lib()
    M, K = A.shape
    N = W.shape[1] if layout == KN else W.shape[0]
    hdr = L.fg_workspace_header_bytes()
    if ws is None:
        ws = torch.full((hdr + 32 * M * N * 4,), 0xFF, dtype=torch.uint8, device=device)
        capi.check(L.fg_workspace_init(ptr(ws), ws.numel(), stream_ptr()), "init")
    C = torch.full((M, N), float("nan"), dtype=torch.half, device=device) if C0 is None else C0.to(device).clone()
    Ad, Wd = A.to(device), W.to(device)     # held until the call has run
    st = L.fg_gemm_f16_planned(ptr(Ad), ptr(Wd), ptr(C), M, N, K, layout, int(accumulate),
                               ctypes.byref(plan), ptr(ws), ws.numel(), stream_ptr())
    capi.check(st, "fg_gemm_f16_planned")
    torch.cuda.synchronize()
    assert int(ws[:hdr].view(torch.int32).abs().sum()) == 0, "workspace header not back to zero"
    return C.cpu().numpy()


@pytest.mark.parametrize("name,layout,kw", FAMILIES, ids=[f[0] for f in FAMILIES])
def test_every_family_completes_through_atomics(device, name, layout, kw):
    K, N = 2176, 384
    for M in (1, 3, 8, 16, 19):
        g = gen(8100 + M)
        A = normal((M, K), g)
        W = normal((K, N) if layout == KN else (N, K), g, 0.05)
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
        C0 = normal((M, N), g, 2.0)
        refa, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout, C=C0.numpy(), accumulate=True)
        for splitk in (2, 5, 17, 31):
            kwargs = dict(kw)
            kwargs.setdefault("waves", 4)
            got = _run(A, W, layout, device, make_plan(splitk=splitk, fused=2, **kwargs))
            assert_close_f16(got, ref, "%s M=%d S=%d" % (name, M, splitk))
            two = _run(A, W, layout, device, make_plan(splitk=splitk, fused=0, **kwargs))
            # exact sum against fp32 sum of the same partials: neighbouring fp16 values, except
            # next to zero where an fp16 step is smaller than the fp32 rounding of the partials
            far = (_ulps(got, two) > 1) & (np.abs(got.astype(np.float32) - two.astype(np.float32)) > 2e-6)
            assert not far.any(), (name, M, splitk)
            again = _run(A, W, layout, device, make_plan(splitk=splitk, fused=2, **kwargs))
            assert (got.view(np.uint16) == again.view(np.uint16)).all()
        got = _run(A, W, layout, device, make_plan(splitk=3, fused=2, **dict(kw, waves=kw.get("waves", 4))),
                   accumulate=True, C0=C0)
        assert_close_f16(got, refa, "%s accumulate M=%d" % (name, M))


@pytest.mark.parametrize("layout", [KN, NK])
def test_exact_integers_are_exact(device, layout):
    # small integers: every partial is an integer, fixed point holds it exactly, so the bits are
    # those of the oracle whatever the split
    g = gen(8200)
    M, N, K = 16, 256, 1024
    A = torch.randint(-3, 4, (M, K), generator=g).half()
    W = torch.randint(-4, 5, (K, N) if layout == KN else (N, K), generator=g).half()
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
    kern = dict(kernel=capi.FG_KERNEL_KN_MFMA, unroll=1) if layout == KN else dict(
        kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=16, unroll=1, waves=8)
    for splitk in (2, 4, 7):
        got = _run(A, W, layout, device, make_plan(splitk=splitk, fused=2, **dict(kern, waves=kern.get("waves", 4))))
        assert (got == ref).all()


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("M", [1, 5, 16])
def test_special_values_keep_their_class(device, layout, M):
    """NaN / inf in the inputs stay in the outputs they belong to; +inf and -inf from different
    K ranges meet as NaN; K-range partials beyond 2^20 of one sign add up to an infinite fp16."""
    K, N = 2048, 256
    g = gen(8300 + M)
    A = normal((M, K), g)
    Wnk = normal((N, K), g, 0.05)
    A[M - 1, 17] = float("nan")             # row M-1
    Wnk[5, 900] = float("inf")              # column 5: +-inf by the sign of A[:, 900]
    Wnk[9, 10] = float("inf")
    Wnk[9, 2000] = float("-inf")            # column 9: the two infinities sit in different K ranges
    A[:, 10] = 1.0
    A[:, 2000] = 1.0
    W = Wnk if layout == NK else Wnk.t().contiguous()
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
    kern = _kernel_for(layout, M)
    for splitk in (2, 4, 8):
        got = _run(A, W, layout, device, make_plan(splitk=splitk, fused=2, **kern))
        assert (np.isnan(got) == np.isnan(ref)).all(), splitk
        inf = np.isinf(ref)
        assert (got[inf] == ref[inf]).all(), splitk
        fin = np.isfinite(ref)
        assert np.isfinite(got[fin]).all()
        assert np.abs(got[fin].astype(np.float32) - ref[fin].astype(np.float32)).max(initial=0.0) < 2e-2
        assert np.isnan(got[M - 1]).all() and np.isnan(got[: M - 1, 9]).all()
    # partials beyond the fixed-point range: all products of column 20 positive, 2048 x 60000 x 4
    Wnk[20, :] = 60000.0
    W = Wnk if layout == NK else Wnk.t().contiguous()
    A2 = torch.full((M, K), 4.0, dtype=torch.half)
    got = _run(A2, W, layout, device, make_plan(splitk=4, fused=2, **kern))
    assert (got[:, 20] == np.inf).all()
    A2 = -A2
    got = _run(A2, W, layout, device, make_plan(splitk=4, fused=2, **kern))
    assert (got[:, 20] == -np.inf).all()


def _kernel_for(layout, M):
    if M == 1:
        return dict(kernel=capi.FG_KERNEL_KN_DOT2, m_block=1, unroll=1, waves=4) if layout == KN else dict(
            kernel=capi.FG_KERNEL_NK_DOT2, tile_n=4, m_block=1, unroll=1, waves=4)
    return dict(kernel=capi.FG_KERNEL_KN_MFMA, unroll=1, waves=4) if layout == KN else dict(
        kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=16, unroll=1, waves=8)


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("M", [1, 6, 16])
def test_huge_partials_of_opposite_sign_cancel(device, layout, M):
    """K-range partials of 2^21 .. 2^24, too large for the fixed-point word, whose sum is a small
    finite number: the result is that number, as in every other completion, not inf or NaN.  All
    values are integers, so every fp32 sum on the way is exact and the comparison is for equality."""
    K, N = 8192, 256
    A = torch.full((M, K), 64.0, dtype=torch.half)
    A[1::2] = 1.0                                  # odd rows: partials of 2^16 .. 2^18, inside the range
    Wnk = torch.zeros((N, K), dtype=torch.half)
    q = K // 4
    cols = torch.arange(N)
    # columns 0 mod 4: +64 on the first half of K, -64 on the second
    c0 = cols[cols % 4 == 0]
    Wnk[c0, : 2 * q] = 64.0
    Wnk[c0, 2 * q:] = -64.0
    # columns 1 mod 4: +64, -32, -32 on three quarters, a few ones on the last (a partial inside the range)
    c1 = cols[cols % 4 == 1]
    Wnk[c1, :q] = 64.0
    Wnk[c1, q: 3 * q] = -32.0
    Wnk[c1, 3 * q + 5: 3 * q + 8] = 1.0
    # columns 2 mod 4: -64 then +64, and a column-dependent remainder inside the first quarter
    c2 = cols[cols % 4 == 2]
    Wnk[c2, : 2 * q] = -64.0
    Wnk[c2, 2 * q:] = 64.0
    Wnk[c2, 3] += (c2 % 5).to(torch.half)
    Wnk[c2, q + 3] += 2.0
    # columns 3 mod 4: one sign only, the sum leaves the fp16 range
    c3 = cols[cols % 4 == 3]
    Wnk[c3, :] = 64.0
    W = Wnk if layout == NK else Wnk.t().contiguous()
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
    assert np.isfinite(ref[:, c0.numpy()]).all() and np.isinf(ref[0, 3])
    assert ref[0, 1] == 64.0 * 3 and ref[0, 2] == 64.0 * (2 + 2)
    kern = _kernel_for(layout, M)
    for splitk in (2, 4, 8, 16):
        for fused in (2, 1, 0):
            got = _run(A, W, layout, device, make_plan(splitk=splitk, fused=fused, **kern))
            assert (got.view(np.uint16) == ref.view(np.uint16)).all(), (splitk, fused)
    # on top of C: the old value joins after the cancellation
    C0 = torch.full((M, N), 3.0, dtype=torch.half)
    refa, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout, C=C0.numpy(), accumulate=True)
    got = _run(A, W, layout, device, make_plan(splitk=4, fused=2, **kern), C0=C0, accumulate=True)
    assert (got.view(np.uint16) == refa.view(np.uint16)).all()


def test_limits_of_the_protocol_are_refused(device):
    L = capi.lib()
    hdr = L.fg_workspace_header_bytes()
    # more arrivals than a word can count
    M, N, K = 4, 256, 8192
    A = torch.zeros((M, K), dtype=torch.half, device=device)
    W = torch.zeros((K, N), dtype=torch.half, device=device)
    C = torch.zeros((M, N), dtype=torch.half, device=device)
    ws = torch.zeros(hdr + 64 * M * N * 4, dtype=torch.uint8, device=device)
    p = make_plan(kernel=capi.FG_KERNEL_KN_MFMA, unroll=1, waves=4, splitk=32, fused=2)
    st = L.fg_gemm_f16_planned(ptr(A), ptr(W), ptr(C), M, N, K, KN, 0, ctypes.byref(p), ptr(ws), ws.numel(),
                               stream_ptr())
    assert st == capi.FG_ERR_UNSUPPORTED
    # more output elements than the header has words for
    M, N, K = 32, 16384, 256
    assert M * N > 262144
    A = torch.zeros((M, K), dtype=torch.half, device=device)
    W = torch.zeros((K, N), dtype=torch.half, device=device)
    C = torch.zeros((M, N), dtype=torch.half, device=device)
    ws = torch.zeros(hdr + 2 * M * N * 4, dtype=torch.uint8, device=device)
    p = make_plan(kernel=capi.FG_KERNEL_KN_MFMA, unroll=1, waves=4, splitk=2, fused=2)
    st = L.fg_gemm_f16_planned(ptr(A), ptr(W), ptr(C), M, N, K, KN, 0, ctypes.byref(p), ptr(ws), ws.numel(),
                               stream_ptr())
    assert st == capi.FG_ERR_UNSUPPORTED
    # the library's own plan stays inside both limits
    for (m, n, k, layout) in ((32, 16384, 4096, KN), (16, 16384, 16384, KN), (1, 1024, 28672, KN), (16, 1024, 16384, NK)):
        q = capi.plan(m, n, k, layout)
        assert q.fused != 2 or (q.splitk <= 31 and m * n <= 262144), q.as_dict()
    torch.cuda.synchronize()
