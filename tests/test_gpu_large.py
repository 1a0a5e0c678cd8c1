"""Weights beyond 4 GiB and beyond 2^31 elements: every byte offset into them needs 64 bits.

The weights are generated on the device; the oracle is evaluated on a spread of output columns
(both ends of N plus a seeded sample), for which the matching weight rows are copied to the host.
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import assert_close_f16, gen, normal

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sg():
    import fastgate_amd

    return fastgate_amd.speedgate


def _cols(N, count, seed):
    rng = np.random.default_rng(seed)
    return np.unique(np.concatenate([np.arange(8), np.arange(N - 8, N), rng.integers(0, N, count)]))


def test_fp16_weights_beyond_4gib_both_layouts(device, sg):
    N, K = 49152, 45056                      # 2.2e9 elements, 4.4 GB
    assert N * K > 2 ** 31
    gd = torch.Generator(device=device)
    gd.manual_seed(4401)
    Wt = torch.empty((N, K), dtype=torch.half, device=device)
    for r0 in range(0, N, 8192):             # filled in slabs: no fp32 copy of the whole matrix
        Wt[r0:r0 + 8192] = (torch.randn((8192, K), device=device, generator=gd) * 0.02).half()
    cols = _cols(N, 96, 1)
    Wsub = np.ascontiguousarray(Wt[torch.from_numpy(cols).to(device)].cpu().numpy())
    results = {}
    for M in (1, 2, 8, 16):
        A = normal((M, K), gen(4400 + M))
        ref, _ = oracle.gemm_f16(A.numpy(), Wsub, oracle.W_NK)
        C = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
        sg.edgemm_m8n128k64x4_bt(A.to(device), Wt, C)
        got = C.cpu().numpy()
        assert np.isfinite(got).all()
        assert_close_f16(got[:, cols], ref, "[N,K] beyond 4 GiB, M=%d" % M)
        results[M] = (A, ref, got)
    Wkn = Wt.t().contiguous()
    del Wt
    for M, (A, ref, got_nk) in results.items():
        C = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
        sg.edgemm_m8n128k64x4(A.to(device), Wkn, C)
        got = C.cpu().numpy()
        assert_close_f16(got[:, cols], ref, "[K,N] beyond 4 GiB, M=%d" % M)
        assert_close_f16(got, got_nk, "layouts agree beyond 4 GiB, M=%d" % M)


def test_int8_weights_beyond_4gib(device, sg):
    N, K = 69632, 65536                      # 4.56e9 bytes
    assert N * K > 2 ** 32
    gd = torch.Generator(device=device)
    gd.manual_seed(4402)
    Wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=device, generator=gd)
    cols = _cols(N, 96, 2)
    Wsub = np.ascontiguousarray(Wq[torch.from_numpy(cols).to(device)].cpu().numpy())
    scale = (torch.rand(N, generator=gen(4403)) * 0.0009 + 0.0001).half()
    ssub = scale.numpy()[cols]
    for M in (1, 2, 8):
        x = normal((M, K), gen(4410 + M))
        y = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
        sg.fastgemv_int8(Wq, x.to(device), y, scale=scale.to(device))
        ref, _ = oracle.gemv_w8a16(Wsub, x.numpy(), ssub)
        got = y.cpu().numpy()
        assert np.isfinite(got).all()
        assert_close_f16(got[:, cols], ref.reshape(M, -1), "W8A16 beyond 4 GiB, M=%d" % M)
    # integer stage, bit for bit
    xq = torch.randint(-127, 128, (1, K), dtype=torch.int8, generator=gen(4420))
    acc = torch.full((1, N), -1, dtype=torch.int32, device=device)
    sg.gemv_i8i8_i32(Wq, xq.to(device), acc)
    acc_ref = oracle.gemv_i8i8_i32(Wsub, xq.numpy())
    assert (acc.cpu().numpy()[:, cols] == acc_ref).all()


def test_int4_weights_beyond_4gib(device, sg):
    N, K = 69632, 131072                     # 4.56e9 bytes of packed nibbles
    assert N * (K // 2) > 2 ** 32
    gd = torch.Generator(device=device)
    gd.manual_seed(4404)
    Wq4 = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, device=device, generator=gd)
    cols = _cols(N, 64, 3)
    Wsub = np.ascontiguousarray(Wq4[torch.from_numpy(cols).to(device)].cpu().numpy())
    scale = (torch.rand(N, generator=gen(4405)) * 0.0009 + 0.0001).half()
    ssub = scale.numpy()[cols]
    for M in (1, 2, 4):
        x = normal((M, K), gen(4430 + M))
        y = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
        sg.fastgemv_int4(Wq4, x.to(device), y, scale=scale.to(device), zero_point=8.0)
        ref, _ = oracle.gemv_w4a16(Wsub, x.numpy(), ssub, 1.0, 8.0)
        got = y.cpu().numpy()
        assert np.isfinite(got).all()
        assert_close_f16(got[:, cols], ref, "W4A16 beyond 4 GiB, M=%d" % M)
