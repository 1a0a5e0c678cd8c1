"""fg_gemm_f16_static (the entry point that allocates nothing: split-K scratch in a static
device array) against fg_gemm_f16 with a caller-allocated workspace, through the C ABI.

Two calls in a row share the GPU's one scratch array, the second with a smaller input, so the
second runs over whatever the first left behind (stale partials beyond its own, counters that
must have returned to zero).  Outputs must agree bit for bit: both entry points run the same
plan and the same kernels, and the split-K sum order is fixed.
"""
import numpy as np
import pytest
import torch

from fastgate_amd import capi
from tests import helpers as h

KN, NK = capi.FG_W_KN, capi.FG_W_NK

# (M, N, K, layout), a larger call followed by a smaller one; every plan splits K across workgroups
PAIRS = [
    ((16, 4096, 4096, KN), (4, 1024, 2048, KN)),
    ((8, 8192, 8192, KN), (1, 2048, 4096, KN)),
    ((16, 2048, 8192, NK), (9, 1024, 8192, NK)),
    ((24, 2048, 4096, KN), (3, 1024, 1024, KN)),  # more than 16 rows: second-pass reduction
]


def _inputs(M, N, K, layout, seed, device):
    g = h.gen(seed)
    A = h.normal((M, K), g).to(device)
    W = h.normal((K, N) if layout == KN else (N, K), g, 0.02).to(device)
    return A, W


def _static(A, W, C, layout, accumulate=False, splitk=0):
    M, K = A.shape
    N = W.shape[1] if layout == KN else W.shape[0]
    st = capi.lib().fg_gemm_f16_static(h.ptr(A), h.ptr(W), h.ptr(C), M, N, K, layout, int(accumulate),
                                       splitk, h.stream_ptr())
    capi.check(st, "fg_gemm_f16_static")


@pytest.mark.gpu
@pytest.mark.parametrize("first,second", PAIRS)
def test_static_scratch_matches_workspace_entry_point(device, first, second):
    for i, (M, N, K, layout) in enumerate((first, second)):
        p = capi.plan(M, N, K, layout)
        assert p.splitk > 1 and p.workspace_bytes <= capi.FG_STATIC_SCRATCH_BYTES, p.as_dict()
        print("fg_gemm_f16_static M=%d N=%d K=%d layout=%d splitk=%d fused=%d" % (M, N, K, layout, p.splitk, p.fused),
              flush=True)
        A, W = _inputs(M, N, K, layout, 4100 + i, device)
        for accumulate in (False, True):
            start = h.normal((M, N), h.gen(77), 1.0).to(device)
            ref = start.clone()
            h.capi_gemm(A, W, ref, layout, accumulate=accumulate)
            got = start.clone()
            _static(A, W, got, layout, accumulate)
            torch.cuda.synchronize()
            assert np.array_equal(got.cpu().numpy().view(np.uint16), ref.cpu().numpy().view(np.uint16)), \
                (M, N, K, layout, accumulate)


@pytest.mark.gpu
def test_static_scratch_unsplit_shapes_and_repeats(device):
    # a plan without a split never touches the scratch array; repeated split calls keep agreeing
    M, N, K = 16, 8192, 8192
    assert capi.plan(M, N, K, NK).splitk == 1
    A, W = _inputs(M, N, K, NK, 4200, device)
    ref = torch.empty((M, N), dtype=torch.half, device=device)
    got = torch.empty_like(ref)
    h.capi_gemm(A, W, ref, NK)
    _static(A, W, got, NK)
    assert torch.equal(got, ref)
    A, W = _inputs(8, 4096, 4096, KN, 4201, device)
    ref = torch.empty((8, 4096), dtype=torch.half, device=device)
    h.capi_gemm(A, W, ref, KN)
    for _ in range(20):
        got = torch.full_like(ref, float("nan"))
        _static(A, W, got, KN)
        assert torch.equal(got, ref)


def test_static_scratch_limit_from_the_plan():
    # host-only: the limit follows from the plan's workspace size; no launching entry point is called
    M, N, K = 16, 16384, 2048
    assert capi.plan(M, N, K, KN, 16).workspace_bytes > capi.FG_STATIC_SCRATCH_BYTES
    assert capi.plan(M, N, K, KN).workspace_bytes <= capi.FG_STATIC_SCRATCH_BYTES
    assert "static" in capi.strerror(capi.FG_ERR_SCRATCH_LIMIT)


@pytest.mark.gpu
def test_static_scratch_rejects_plans_beyond_its_limit(device):
    L = capi.lib()
    M, N, K = 16, 16384, 2048
    A, W = _inputs(M, N, K, KN, 4300, device)
    C = torch.full((M, N), 7.0, dtype=torch.half, device=device)
    st = L.fg_gemm_f16_static(h.ptr(A), h.ptr(W), h.ptr(C), M, N, K, KN, 0, 16, h.stream_ptr())
    assert st == capi.FG_ERR_SCRATCH_LIMIT
    torch.cuda.synchronize()
    assert bool((C == 7.0).all())          # refused before any device work
    # the library's own plan for the same shape fits and runs
    ref = torch.empty_like(C)
    h.capi_gemm(A, W, ref, KN)
    _static(A, W, C, KN)
    assert torch.equal(C, ref)
