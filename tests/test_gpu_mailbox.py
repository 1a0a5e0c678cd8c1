"""Split-K completion of the [K,N] MFMA kernel through flags in one XCD's L2 (plan.fused = 3):
against the oracle, bit for bit against the second-kernel and counter completions, with a fifth of
the workgroups claiming to run on another XCD (plan.fused = 4: the recomputing path), on a shared
workspace across changing shapes, on two streams, and replayed from a captured graph."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from fastgate_amd import capi
from helpers import assert_close_f16, gen, make_plan, normal, ptr, stream_ptr

pytestmark = pytest.mark.gpu

KN = capi.FG_W_KN


def _workspace(device, mib=24):
    L = capi.lib()
    ws = torch.full((L.fg_workspace_header_bytes() + (mib << 20),), 0xFF, dtype=torch.uint8, device=device)
    capi.check(L.fg_workspace_init(ptr(ws), ws.numel(), stream_ptr()), "init")
    return ws


def _call(Ad, Wd, C, plan, ws, accumulate=False, stream=None):
    L = capi.lib()
    M, K = Ad.shape
    N = Wd.shape[1]
    st = L.fg_gemm_f16_planned(ptr(Ad), ptr(Wd), ptr(C), M, N, K, KN, int(accumulate), ctypes.byref(plan),
                               ptr(ws), ws.numel(), stream if stream is not None else stream_ptr())
    capi.check(st, "fg_gemm_f16_planned")


def _plan(splitk, fused, waves=4, unroll=1):
    return make_plan(capi.FG_KERNEL_KN_MFMA, m_block=16, waves=waves, unroll=unroll, splitk=splitk, fused=fused)


def _bits(t):
    return t.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("waves,unroll", [(4, 1), (8, 1), (4, 2), (8, 2)])
def test_mailbox_matches_oracle_and_other_completions(device, waves, unroll):
    ws = _workspace(device)
    # N = 384: three column tiles, fewer than XCDs (most of the padded grid has no work);
    # N = 1408: eleven tiles, two on some XCDs and one on others
    for N, K in ((384, 2176), (1408, 1024)):
        for M in (1, 3, 8, 16, 19):
            g = gen(9100 + M + N)
            A, W = normal((M, K), g), normal((K, N), g, 0.05)
            ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), KN)
            C0 = normal((M, N), g, 2.0)
            refa, _ = oracle.gemm_f16(A.numpy(), W.numpy(), KN, C=C0.numpy(), accumulate=True)
            Ad, Wd = A.to(device), W.to(device)
            for splitk in (2, 5, 8, 17, 32):
                if (K // 32) < splitk * waves * unroll and splitk > 8:
                    continue   # fewer K units than wave slots: still legal, covered by the smaller splits
                out = {}
                for fused in (0, 1, 3, 4):
                    C = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
                    _call(Ad, Wd, C, _plan(splitk, fused, waves, unroll), ws)
                    out[fused] = _bits(C)
                assert_close_f16(out[3].view(np.float16), ref, "mailbox M=%d N=%d S=%d" % (M, N, splitk))
                for fused in (0, 1, 4):
                    assert (out[3] == out[fused]).all(), (M, N, splitk, fused)
            for fused in (3, 4):
                C = C0.to(device).clone()
                _call(Ad, Wd, C, _plan(3, fused, waves, unroll), ws, accumulate=True)
                assert_close_f16(C.cpu().numpy(), refa, "mailbox accumulate M=%d fused=%d" % (M, fused))
    hdr = capi.lib().fg_workspace_header_bytes()
    flags_at = 65536 + 262144 * 12
    assert hdr == flags_at + 65536 * 8
    torch.cuda.synchronize()
    # counters and accumulator words are back at zero; the flag words keep launch tags
    assert int(ws[:flags_at].view(torch.int32).abs().sum()) == 0
    assert int(ws[flags_at:hdr].view(torch.int64).ne(0).sum()) > 0


def test_mailbox_shared_workspace_changing_shapes_and_streams(device):
    """Flags of earlier launches (other shapes, other splits, another stream) must never count."""
    ws = _workspace(device)
    g = gen(9200)
    cases = []
    for (M, N, K, S) in ((16, 1024, 2048, 8), (8, 2048, 1024, 4), (16, 1024, 2048, 16), (5, 384, 4096, 8),
                         (16, 1024, 2048, 8), (12, 3072, 512, 2)):
        A, W = normal((M, K), g), normal((K, N), g, 0.05)
        ref = (A.float() @ W.float()).half().numpy()
        cases.append((A.to(device), W.to(device), ref, S))
    side = torch.cuda.Stream()
    for rep in range(6):
        for i, (Ad, Wd, ref, S) in enumerate(cases):
            C = torch.full((Ad.shape[0], Wd.shape[1]), float("nan"), dtype=torch.half, device=device)
            if (rep + i) % 3 == 2:
                # same workspace from a second stream, ordered by events as the header asks for
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    _call(Ad, Wd, C, _plan(S, 3), ws, stream=ctypes.c_void_p(side.cuda_stream))
                torch.cuda.current_stream().wait_stream(side)
            else:
                _call(Ad, Wd, C, _plan(S, 3 if rep % 2 == 0 else 4), ws)
            C1 = torch.full_like(C, float("nan"))
            _call(Ad, Wd, C1, _plan(S, 1), ws)
            torch.cuda.synchronize()
            assert_close_f16(C.cpu().numpy(), ref, "rep %d case %d" % (rep, i))
            assert (_bits(C) == _bits(C1)).all(), (rep, i)


def test_mailbox_under_graph_replay(device):
    """A captured launch keeps its kernel arguments: every replay must still get its own tag.  The
    inputs change between replays; each replay is checked against an eager call."""
    ws = _workspace(device)
    g = gen(9300)
    M, N, K, S = 16, 2048, 2048, 8
    Ad = normal((M, K), g).to(device)
    Wd = normal((K, N), g, 0.05).to(device)
    C = torch.zeros((M, N), dtype=torch.half, device=device)
    plan = _plan(S, 3)
    _call(Ad, Wd, C, plan, ws)           # first use outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _call(Ad, Wd, C, plan, ws, stream=ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    for rep in range(5):
        Ad.copy_(normal((M, K), g).to(device))
        C.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = _bits(C).copy()
        Ce = torch.full_like(C, float("nan"))
        _call(Ad, Wd, Ce, _plan(S, 0), ws)
        torch.cuda.synchronize()
        assert (got == _bits(Ce)).all(), rep
        assert_close_f16(got.view(np.float16), (Ad.float() @ Wd.float()).half().cpu().numpy(), "replay %d" % rep)


def test_mailbox_limits(device):
    L = capi.lib()
    ws = _workspace(device, 4)
    A = torch.zeros((4, 4096), dtype=torch.half, device=device)
    W = torch.zeros((4096, 256), dtype=torch.half, device=device)
    C = torch.zeros((4, 256), dtype=torch.half, device=device)
    # 33 partners do not fit the owner's mask; other kernel families have no such completion
    p = _plan(33, 3)
    st = L.fg_gemm_f16_planned(ptr(A), ptr(W), ptr(C), 4, 256, 4096, KN, 0, ctypes.byref(p), ptr(ws), ws.numel(), stream_ptr())
    assert st == capi.FG_ERR_UNSUPPORTED
    p = make_plan(capi.FG_KERNEL_KN_DOT2, m_block=4, splitk=4, fused=3)
    st = L.fg_gemm_f16_planned(ptr(A), ptr(W), ptr(C), 4, 256, 4096, KN, 0, ctypes.byref(p), ptr(ws), ws.numel(), stream_ptr())
    assert st == capi.FG_ERR_UNSUPPORTED
    p = _plan(4, 5)
    st = L.fg_gemm_f16_planned(ptr(A), ptr(W), ptr(C), 4, 256, 4096, KN, 0, ctypes.byref(p), ptr(ws), ws.numel(), stream_ptr())
    assert st == capi.FG_ERR_INVALID_ARG
    torch.cuda.synchronize()


def test_mailbox_fast_path_whatever_xcd_the_dispatch_starts_on(device):
    """The XCD that workgroup 0 of a launch lands on depends on what ran before.  The partners of
    a tile must still find each other: after launches of assorted grid sizes the mailbox call may
    not fall back to recomputing its partners' K ranges, which costs several times the call.  The
    bound is loose (2.5x the counter completion; the fallback measured 4x) and results are checked
    bit for bit as well."""
    L = capi.lib()
    ws = _workspace(device)
    g = gen(9400)
    M, N, K, S = 16, 4096, 4096, 8
    Ad, Wd = normal((M, K), g).to(device), normal((K, N), g, 0.05).to(device)
    C1 = torch.zeros((M, N), dtype=torch.half, device=device)
    C3 = torch.zeros_like(C1)
    Ks = 1024
    As = normal((4, Ks), g).to(device)

    def shift(tiles, split):
        # a [K,N] call of tiles x split workgroups in plain order moves the starting XCD of what follows
        Ws = torch.zeros((Ks, 128 * tiles), dtype=torch.half, device=device)
        Cs = torch.zeros((4, 128 * tiles), dtype=torch.half, device=device)
        _call(As, Ws, Cs, make_plan(capi.FG_KERNEL_KN_DOT2, m_block=4, waves=4, splitk=split, fused=1 if split > 1 else 0), ws)

    def timed(plan, C, reps=30):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            _call(Ad, Wd, C, plan, ws)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    for tiles, split in ((1, 1), (1, 3), (1, 5), (1, 7), (43, 2), (37, 7), (129, 4), (17, 13), (3, 3)):
        shift(tiles, split)
        timed(_plan(S, 1), C1, 5)
        shift(tiles, split)
        t3 = timed(_plan(S, 3), C3)
        shift(tiles, split)
        t1 = timed(_plan(S, 1), C1)
        assert (_bits(C1) == _bits(C3)).all(), (tiles, split)
        assert t3 < 2.5 * t1, (tiles, split, t3, t1)
