"""Shared test utilities: seeded inputs of the benchmark configurations, the tolerance the
path is held to, and thin callers of the C ABI that take torch tensors."""
from __future__ import annotations

import ctypes

import numpy as np
import torch

from fastgate_amd import capi

# fp16 outputs: |y - ref| <= ATOL + RTOL * |ref| against the fp32-accumulate oracle.
ATOL = 1e-2
RTOL = 2e-3


def gen(seed: int):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def uniform_pm1(shape, g):
    return (torch.rand(shape, generator=g) * 2 - 1).half()


def normal(shape, g, std=1.0):
    return (torch.randn(shape, generator=g) * std).half()


def assert_close_f16(got, ref, what=""):
    """got, ref: float16 numpy arrays of the same shape."""
    got = np.asarray(got, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    err = np.abs(got - ref)
    tol = ATOL + RTOL * np.abs(ref)
    bad = err > tol
    if bad.any() or not np.isfinite(got).all():
        idx = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(
            "%s: %d of %d outside |d| <= %.0e + %.0e|ref|; worst at %s got %r ref %r"
            % (what, int(bad.sum()), bad.size, ATOL, RTOL, idx, got[idx], ref[idx]))


def stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def capi_gemm(A, W, C, w_layout, accumulate=False, splitk=0, plan=None):
    """fg_gemm_f16 / fg_gemm_f16_planned on device tensors; allocates the workspace the plan
    asks for.  Returns the plan used."""
    L = capi.lib()
    M, K = A.shape
    N = W.shape[1] if w_layout == capi.FG_W_KN else W.shape[0]
    hdr = L.fg_workspace_header_bytes()
    if plan is None:
        p = capi.plan(M, N, K, w_layout, splitk)
        wsb = p.workspace_bytes
    else:
        p = plan
        # the transposing kernel derives its split from K; leave room for any split up to K/128
        wsb = hdr + max(p.splitk, K // 128) * M * N * 4
    ws = None
    if wsb:
        # poisoned partials, then the counter header zeroed through the C ABI
        ws = torch.full((wsb,), 0xFF, dtype=torch.uint8, device=A.device)
        capi.check(L.fg_workspace_init(ptr(ws), wsb, stream_ptr()), "fg_workspace_init")
    if plan is None:
        st = L.fg_gemm_f16(ptr(A), ptr(W), ptr(C), M, N, K, w_layout, int(accumulate), splitk,
                           ptr(ws), wsb, stream_ptr())
    else:
        st = L.fg_gemm_f16_planned(ptr(A), ptr(W), ptr(C), M, N, K, w_layout, int(accumulate),
                                   ctypes.byref(p), ptr(ws), wsb, stream_ptr())
    capi.check(st, "fg_gemm_f16")
    return p


def make_plan(kernel, tile_n=0, m_block=0, waves=4, unroll=1, splitk=1, stream_w=1, fused=1, stagger=0, band=0):
    p = capi.Plan()
    p.kernel, p.tile_n, p.m_block, p.waves = kernel, tile_n, m_block, waves
    p.unroll, p.splitk, p.stream_w, p.fused, p.stagger = unroll, splitk, stream_w, fused, stagger
    p.band = band
    return p
