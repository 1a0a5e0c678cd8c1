"""Non-finite and extreme values: NaN / inf in the inputs stay in the outputs they belong to,
fp16 overflow of a sum becomes inf, subnormal inputs are multiplied (not flushed), exactly as the
CPU oracle (fp16 products, fp32 accumulation) has it."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from fastgate_amd import capi
from helpers import assert_close_f16, capi_gemm, gen, normal, ptr, stream_ptr

pytestmark = pytest.mark.gpu

KN, NK = capi.FG_W_KN, capi.FG_W_NK


def _gemm(A, W, layout, device):
    M = A.shape[0]
    N = W.shape[1] if layout == KN else W.shape[0]
    C = torch.zeros((M, N), dtype=torch.half, device=device)
    capi_gemm(A.to(device), W.to(device), C, layout)
    torch.cuda.synchronize()
    return C.cpu().numpy()


def _same_class(got, ref):
    """NaN where ref is NaN, the same inf where ref is inf, finite elsewhere."""
    assert (np.isnan(got) == np.isnan(ref)).all()
    inf = np.isinf(ref)
    assert (got[inf] == ref[inf]).all()
    assert np.isfinite(got[~inf & ~np.isnan(ref)]).all()


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("M", [1, 2, 5, 8, 16])
def test_nan_and_inf_stay_in_their_row_and_column(device, layout, M):
    K, N = 1152, 384
    g = gen(700 + M)
    A = normal((M, K), g)
    Wnk = normal((N, K), g, 0.05)
    A[M - 1, 17] = float("nan")            # poisons output row M-1 only
    Wnk[5, 900] = float("inf")             # poisons output column 5 (sign follows A[:, 900])
    Wnk[300, 3] = float("-inf")
    Wnk[301, 10] = float("inf")
    Wnk[301, 11] = float("-inf")           # inf - inf (unless A is 0 there): NaN in column 301
    W = Wnk if layout == NK else Wnk.t().contiguous()
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
    got = _gemm(A, W, layout, device)
    _same_class(got, ref)
    assert np.isnan(got[M - 1]).all()
    clean = np.ones(N, bool)
    clean[[5, 300, 301]] = False
    fin = np.isfinite(ref)
    assert fin[: M - 1][:, clean].all()
    assert np.abs(got[fin].astype(np.float32) - ref[fin].astype(np.float32)).max(initial=0.0) < 2e-2


@pytest.mark.parametrize("layout", [KN, NK])
def test_overflow_of_the_sum_is_inf_and_subnormals_count(device, layout):
    K, N, M = 256, 128, 3
    # 256 products of 60000 * 1 overflow fp16 (65504) but not fp32: +-inf after the final rounding
    A = torch.ones((M, K), dtype=torch.half)
    A[1] = -1.0
    A[2, 1:] = 0.0                          # row 2 sees a single product: finite
    Wnk = torch.full((N, K), 60000.0, dtype=torch.half)
    W = Wnk if layout == NK else Wnk.t().contiguous()
    got = _gemm(A, W, layout, device)
    assert (got[0] == np.inf).all() and (got[1] == -np.inf).all() and (got[2] == 60000.0).all()
    # subnormal weights (2^-24) times 2^10 activations: 256 * 2^-14 = 2^-6, exact
    sub = torch.tensor(np.full((N, K), 1, np.uint16).view(np.float16))   # smallest subnormal
    W = sub if layout == NK else sub.t().contiguous()
    A = torch.full((M, K), 1024.0, dtype=torch.half)
    got = _gemm(A, W, layout, device)
    assert (got == np.float16(2.0 ** -6)).all()


def test_int8_gemv_with_non_finite_activations(device):
    L = capi.lib()
    N, K = 256, 512
    g = gen(720)
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    Wq[:, 7] = 0                            # a zero weight times inf is NaN, as in the oracle
    for M in (1, 2, 4, 8):
        x = normal((M, K), g)
        x[0, 7] = float("inf")
        x[M - 1, 100] = float("nan")
        ref, _ = oracle.gemv_w8a16(Wq.numpy(), x.numpy(), None, 1.0, 0.0)
        y = torch.zeros((M, N), dtype=torch.half, device=device)
        Wd, xd = Wq.to(device), x.to(device)
        capi.check(L.fg_gemv_w8a16(ptr(Wd), ptr(xd), None, 1.0, 0.0, ptr(y), M, N, K, stream_ptr()), "w8a16")
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        _same_class(got, ref.reshape(M, N))
        assert np.isnan(got[0]).all() and np.isnan(got[M - 1]).all()


# ---------------------------------------------------------------------------------------
# [K,N] weights with padded rows
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("M", [1, 2, 5, 16])
@pytest.mark.parametrize("N,K,pad", [(512, 1152, 8), (1024, 640, 128), (2048, 4096, 136)])
def test_pitched_kn_weights_match_the_dense_call_bit_for_bit(device, M, N, K, pad):
    import fastgate_amd

    sg = fastgate_amd.speedgate
    g = gen(9100 + M + N + pad)
    A = normal((M, K), g)
    W = normal((K, N), g, 0.05)
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), oracle.W_KN)
    padded = torch.full((K, N + pad), float("nan"), dtype=torch.half, device=device)
    padded[:, :N] = W.to(device)
    view = padded[:, :N]
    assert not view.is_contiguous() and view.stride(0) == N + pad
    Ad = A.to(device)
    dense = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
    pitched = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
    sg.edgemm_m8n128k64x4(Ad, W.to(device), dense)
    sg.edgemm_m8n128k64x4(Ad, view, pitched)
    assert_close_f16(pitched.cpu().numpy(), ref, "pitch %d" % (N + pad))
    assert (pitched.cpu().numpy().view(np.uint16) == dense.cpu().numpy().view(np.uint16)).all()
    # accumulate protocol through a flat_gemm name
    acc = torch.ones((M, N), dtype=torch.half, device=device)
    sg.flat_gemm_m8n128k64x4_bz1(Ad, view, acc, 0)
    ref_acc, _ = oracle.gemm_f16(A.numpy(), W.numpy(), oracle.W_KN, C=np.ones((M, N), np.float16),
                                 accumulate=True)
    assert_close_f16(acc.cpu().numpy(), ref_acc, "accumulate, pitch %d" % (N + pad))


def test_pitched_entry_point_rejects_bad_pitches(device):
    L = capi.lib()
    M, N, K = 4, 256, 256
    A = torch.zeros((M, K), dtype=torch.half, device=device)
    W = torch.zeros((K, N + 64), dtype=torch.half, device=device)
    C = torch.zeros((M, N), dtype=torch.half, device=device)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=device)
    args = lambda ldw: (ptr(A), ptr(W), ptr(C), M, N, K, ldw, 0, 0, ptr(ws), ws.numel(), stream_ptr())
    assert L.fg_gemm_f16_pitched(*args(N + 64)) == capi.FG_OK
    assert L.fg_gemm_f16_pitched(*args(N - 8)) == capi.FG_ERR_INVALID_ARG      # rows overlap
    assert L.fg_gemm_f16_pitched(*args(N + 4)) == capi.FG_ERR_INVALID_ARG      # not 16-byte rows
    torch.cuda.synchronize()


@pytest.mark.parametrize("layout,M,N,K", [(KN, 9, 7168, 2048), (KN, 1, 11008, 8192), (KN, 16, 4096, 4096),
                                          (NK, 16, 3072, 12288)])
def test_in_launch_split_k_repeats_bit_for_bit(device, layout, M, N, K):
    """A completion that races shows as a rare wrong sum.  Several hundred back-to-back calls on
    rotating weights must all give the same bits.  With the counter protocol (every wave's partial
    has to be in memory before its workgroup arrives at the tile counter) those are the bits of
    the two-pass completion, where a second kernel sums the same partials in the same order; the
    atomic protocol sums in fixed point, so it is held to its own first result, and that result to
    the two-pass one within one fp16 ulp."""
    L = capi.lib()
    p = capi.plan(M, N, K, layout, 0)
    if p.splitk < 2 or not p.fused:
        pytest.skip("the library does not split this shape inside the launch")
    g = torch.Generator(device=device).manual_seed(4242 + N + K)
    shape = (K, N) if layout == KN else (N, K)
    Ws = [(torch.randn(shape, device=device, generator=g) * 0.02).half() for _ in range(4)]
    A = torch.randn((M, K), device=device, generator=g).half()
    ws = torch.zeros(p.workspace_bytes, dtype=torch.uint8, device=device)
    two = capi.plan(M, N, K, layout, 0)
    two.fused = 0
    refs = []
    for W in Ws:
        C = torch.empty((M, N), dtype=torch.half, device=device)
        capi.check(L.fg_gemm_f16_planned(ptr(A), ptr(W), ptr(C), M, N, K, layout, 0, ctypes.byref(two), ptr(ws),
                                         ws.numel(), stream_ptr()), "two-pass")
        refs.append(C)
    assert_close_f16(refs[0].cpu().numpy(), (A.float() @ (Ws[0].float() if layout == KN else Ws[0].float().t())).cpu().numpy(),
                     "two-pass reference")
    for protocol in sorted({1, p.fused}):
        q = capi.plan(M, N, K, layout, 0)
        q.fused = protocol
        want = refs
        if protocol == 2:
            want = []
            for i, W in enumerate(Ws):
                C = torch.empty((M, N), dtype=torch.half, device=device)
                capi.check(L.fg_gemm_f16_planned(ptr(A), ptr(W), ptr(C), M, N, K, layout, 0, ctypes.byref(q),
                                                 ptr(ws), ws.numel(), stream_ptr()), "atomic")
                want.append(C)
                a = C.cpu().numpy().view(np.int16).astype(np.int32)
                b = refs[i].cpu().numpy().view(np.int16).astype(np.int32)
                far = (np.abs(a - b) > 1) & ((C.float() - refs[i].float()).abs().cpu().numpy() > 2e-6)
                assert not far.any()                # neighbouring fp16 values, except next to zero
        C = torch.empty((M, N), dtype=torch.half, device=device)
        bad = torch.zeros((), dtype=torch.int64, device=device)
        for i in range(400):
            capi.check(L.fg_gemm_f16_planned(ptr(A), ptr(Ws[i % 4]), ptr(C), M, N, K, layout, 0, ctypes.byref(q),
                                             ptr(ws), ws.numel(), stream_ptr()), "in-launch")
            bad += (C.view(torch.int16) != want[i % 4].view(torch.int16)).sum()
        assert int(bad.item()) == 0, protocol
    # and through the entry point that plans by itself
    C = torch.empty((M, N), dtype=torch.half, device=device)
    capi.check(L.fg_gemm_f16(ptr(A), ptr(Ws[0]), ptr(C), M, N, K, layout, 0, 0, ptr(ws), ws.numel(),
                             stream_ptr()), "planned by the library")
    assert torch.equal(C, want[0] if p.fused == 2 else refs[0])
