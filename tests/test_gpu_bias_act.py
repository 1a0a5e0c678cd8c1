"""GPU parity of the fused bias + activation tail (fg_gemm_f16_bias_act and the pybind operators
built on it) against the CPU oracle: every kernel family, with and without split-K, finished in
the launch or by the second-pass kernel."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from fastgate_amd import capi
from helpers import assert_close_f16, gen, make_plan, normal, ptr, stream_ptr

pytestmark = pytest.mark.gpu

KN, NK = capi.FG_W_KN, capi.FG_W_NK
ACTS = ["none", "relu", "gelu", "gelu_tanh", "silu"]


def _bias_act(A, W, bias, act, layout, device, plan=None, splitk=0):
    L = capi.lib()
    M, K = A.shape
    N = W.shape[1] if layout == KN else W.shape[0]
    Ad, Wd = A.to(device), W.to(device)
    bd = None if bias is None else bias.to(device)
    C = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
    wsb = L.fg_workspace_header_bytes() + max(K // 128, 64) * M * N * 4
    ws = torch.full((wsb,), 0xFF, dtype=torch.uint8, device=device)
    capi.check(L.fg_workspace_init(ptr(ws), wsb, stream_ptr()), "fg_workspace_init")
    st = L.fg_gemm_f16_bias_act(ptr(Ad), ptr(Wd), ptr(bd), capi.ACT_IDS[act], ptr(C), M, N, K, layout,
                                splitk, None if plan is None else ctypes.byref(plan), ptr(ws), wsb,
                                stream_ptr())
    capi.check(st, "fg_gemm_f16_bias_act")
    torch.cuda.synchronize()
    return C.cpu().numpy()


def _plans():
    return [
        ("nk_dot2", NK, dict(kernel=capi.FG_KERNEL_NK_DOT2, tile_n=4, m_block=2, unroll=2)),
        ("nk_mfma4", NK, dict(kernel=capi.FG_KERNEL_NK_MFMA4, tile_n=16, m_block=8, unroll=1)),
        ("nk_mfma_r", NK, dict(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=16, unroll=1, waves=8)),
        ("kn_dot2", KN, dict(kernel=capi.FG_KERNEL_KN_DOT2, m_block=2, unroll=2)),
        ("kn_mfma", KN, dict(kernel=capi.FG_KERNEL_KN_MFMA, unroll=1)),
    ]


@pytest.mark.parametrize("name,layout,kw", _plans(), ids=[p[0] for p in _plans()])
@pytest.mark.parametrize("splitk,fused", [(1, 0), (3, 1), (2, 0), (3, 2)])
def test_every_kernel_family(device, name, layout, kw, splitk, fused):
    K, N = 1152, 384
    for M in (1, 7, 16, 19):
        g = gen(300 + M)
        A = normal((M, K), g)
        W = normal((K, N) if layout == KN else (N, K), g, 0.05)
        bias = normal((N,), g, 1.5)
        for i, act in enumerate(ACTS):
            b = None if (i + M) % 3 == 0 else bias
            ref = oracle.gemm_bias_act(A.numpy(), W.numpy(), layout, None if b is None else b.numpy(), act)
            kwargs = dict(kw)
            kwargs.update(splitk=splitk, fused=fused)
            got = _bias_act(A, W, b, act, layout, device, plan=make_plan(**kwargs))
            assert_close_f16(got, ref, "%s M=%d act=%s bias=%s S=%d fused=%d" % (name, M, act, b is not None, splitk, fused))


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("M", [1, 2, 4, 8, 16, 24])
def test_library_plans_at_ffn_shapes(device, layout, M):
    # scaled-down feed-forward pair (K:N = 1:4 and 4:1): the planner's own choices
    for K, N in ((768, 3072), (3072, 768)):
        g = gen(310 + M + K)
        A = normal((M, K), g)
        W = normal((K, N) if layout == KN else (N, K), g, 0.03)
        bias = normal((N,), g, 1.0)
        for act in ("gelu", "silu"):
            ref = oracle.gemm_bias_act(A.numpy(), W.numpy(), layout, bias.numpy(), act)
            assert_close_f16(_bias_act(A, W, bias, act, layout, device), ref, "auto plan %s" % act)
            ref = oracle.gemm_bias_act(A.numpy(), W.numpy(), layout, bias.numpy(), act)
            assert_close_f16(_bias_act(A, W, bias, act, layout, device, splitk=4), ref, "split 4 %s" % act)


def test_plain_call_is_unchanged_and_none_tail_matches_it_bitwise(device):
    from helpers import capi_gemm
    for layout in (KN, NK):
        g = gen(320 + layout)
        A = normal((8, 2048), g)
        W = normal((2048, 1024) if layout == KN else (1024, 2048), g, 0.02)
        C = torch.empty((8, 1024), dtype=torch.half, device=device)
        capi_gemm(A.to(device), W.to(device), C, layout)
        torch.cuda.synchronize()
        got = _bias_act(A, W, None, "none", layout, device)
        assert (got.view(np.uint16) == C.cpu().numpy().view(np.uint16)).all()
        # bias of zeros and relu on a non-negative product change nothing either
        Wp = W.abs()
        Ap = A.abs()
        capi_gemm(Ap.to(device), Wp.to(device), C, layout)
        torch.cuda.synchronize()
        got = _bias_act(Ap, Wp, torch.zeros(1024, dtype=torch.half), "relu", layout, device)
        assert (got.view(np.uint16) == C.cpu().numpy().view(np.uint16)).all()


def test_closed_forms(device):
    # A = 0: the output is act(bias) in every row, exactly for relu / none
    N, K = 256, 256
    bias = torch.linspace(-4, 4, N).half()
    A = torch.zeros((5, K), dtype=torch.half)
    W = normal((N, K), gen(330))
    got = _bias_act(A, W, bias, "none", NK, device)
    assert (got == bias.numpy()[None, :]).all()
    got = _bias_act(A, W, bias, "relu", NK, device)
    assert (got == np.maximum(bias.numpy(), 0)[None, :]).all()
    want = torch.nn.functional.gelu(bias.double()).half().numpy()
    assert_close_f16(_bias_act(A, W, bias, "gelu", NK, device), np.repeat(want[None], 5, 0), "gelu(bias)")
    want = torch.nn.functional.silu(bias.double()).half().numpy()
    assert_close_f16(_bias_act(A, W, bias, "silu", NK, device), np.repeat(want[None], 5, 0), "silu(bias)")
    want = torch.nn.functional.gelu(bias.double(), approximate="tanh").half().numpy()
    assert_close_f16(_bias_act(A, W, bias, "gelu_tanh", NK, device), np.repeat(want[None], 5, 0), "gelu_tanh(bias)")


def test_pybind_operators_and_ffn_pair(device):
    import fastgate_amd
    sg = fastgate_amd.speedgate
    g = gen(340)
    M, K, N1 = 16, 768, 3072
    A = normal((M, K), g)
    W1t = normal((N1, K), g, 0.03)
    b1 = normal((N1,), g, 0.5)
    W2t = normal((K, N1), g, 0.03)
    b2 = normal((K,), g, 0.5)
    H = torch.full((M, N1), float("nan"), dtype=torch.half, device=device)
    C = torch.full((M, K), float("nan"), dtype=torch.half, device=device)
    sg.ffn_bt(A.to(device), W1t.to(device), b1.to(device), W2t.to(device), b2.to(device), H, C, act="gelu")
    h_ref = oracle.gemm_bias_act(A.numpy(), W1t.numpy(), NK, b1.numpy(), "gelu")
    assert_close_f16(H.cpu().numpy(), h_ref, "ffn hidden")
    # the down-projection is checked on the hidden activations the GPU produced
    c_ref = oracle.gemm_bias_act(H.cpu().numpy(), W2t.numpy(), NK, b2.numpy(), "none")
    assert_close_f16(C.cpu().numpy(), c_ref, "ffn output")
    # against torch on the device: same pair, unfused
    h_t = torch.nn.functional.gelu(A.to(device).float() @ W1t.to(device).float().t() + b1.to(device).float())
    assert_close_f16(H.cpu().numpy(), h_t.half().cpu().numpy(), "ffn hidden vs torch")
    # [K,N] operator, no bias
    C2 = torch.empty((M, N1), dtype=torch.half, device=device)
    sg.gemm_bias_act(A.to(device), W1t.t().contiguous().to(device), C2, None, "silu")
    ref = oracle.gemm_bias_act(A.numpy(), W1t.numpy(), NK, None, "silu")
    assert_close_f16(C2.cpu().numpy(), ref, "gemm_bias_act silu")
    sg.gemm_bias_act_bt(A.to(device), W1t.to(device), C2, b1.to(device))
    ref = oracle.gemm_bias_act(A.numpy(), W1t.numpy(), NK, b1.numpy(), "none")
    assert_close_f16(C2.cpu().numpy(), ref, "gemm_bias_act_bt bias only")
    with pytest.raises(ValueError):
        sg.gemm_bias_act_bt(A.to(device), W1t.to(device), C2, b1.to(device), "swish")
    with pytest.raises(RuntimeError):
        sg.gemm_bias_act_bt(A.to(device), W1t.to(device), C2, b1[:100].contiguous().to(device), "relu")
    L = capi.lib()
    Ad, Wd = A.to(device), W1t.to(device)
    assert L.fg_gemm_f16_bias_act(ptr(Ad), ptr(Wd), None, 9, ptr(C2), M, N1, K, NK, 0, None, None, 0,
                                  stream_ptr()) == capi.FG_ERR_INVALID_ARG
