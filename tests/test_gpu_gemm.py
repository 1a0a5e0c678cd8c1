"""GPU parity of the fp16 GEMM/GEMV kernels against the CPU oracle, through the C ABI
(ctypes) and through the pybind11 operator surface."""
import numpy as np
import pytest
import torch

import oracle
from fastgate_amd import capi
from helpers import assert_close_f16, capi_gemm, gen, make_plan, normal, uniform_pm1

pytestmark = pytest.mark.gpu

KN, NK = capi.FG_W_KN, capi.FG_W_NK


def _case(M, N, K, layout, seed, wstd=0.02):
    g = gen(seed)
    A = normal((M, K), g)
    W = normal((K, N) if layout == KN else (N, K), g, wstd)
    return A, W


def _run(A, W, layout, device, accumulate=False, C0=None, plan=None, splitk=0):
    M = A.shape[0]
    N = W.shape[1] if layout == KN else W.shape[0]
    Ad, Wd = A.to(device), W.to(device)
    if C0 is None:
        Cd = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
    else:
        Cd = C0.to(device).clone()
    p = capi_gemm(Ad, Wd, Cd, layout, accumulate=accumulate, splitk=splitk, plan=plan)
    torch.cuda.synchronize()
    return Cd.cpu().numpy(), p


# Every kernel family x tile x unroll x waves x split-K on one small ragged-ish shape
# (K = 640 = 5*128 leaves partial steps in every unroll setting).
def _all_plans():
    plans = []
    for mb in (1, 2, 4, 8):
        for rn in (4, 8, 16):
            for u in (1, 2, 4):
                if mb * rn <= 64 and rn * u <= 32:
                    plans.append(("nk_dot2", NK, dict(kernel=capi.FG_KERNEL_NK_DOT2, tile_n=rn, m_block=mb, unroll=u)))
    for mb in (4, 8, 12, 16):
        for tn in (4, 8, 16, 32):
            for u in (1, 2, 4):
                mg, r4 = mb // 4, tn // 4
                if mg * r4 <= 16 and (mg + r4) * u <= 24:
                    plans.append(("nk_mfma4", NK, dict(kernel=capi.FG_KERNEL_NK_MFMA4, tile_n=tn, m_block=mb, unroll=u)))
    for mb in (1, 2, 4, 8):
        for u in (1, 2, 4):
            if not (mb == 8 and u == 4):
                plans.append(("kn_dot2", KN, dict(kernel=capi.FG_KERNEL_KN_DOT2, m_block=mb, unroll=u)))
    for u in (1, 2, 4):
        plans.append(("kn_mfma", KN, dict(kernel=capi.FG_KERNEL_KN_MFMA, unroll=u)))
    return plans


@pytest.mark.parametrize("name,layout,kw", _all_plans(), ids=lambda v: str(v) if not isinstance(v, dict) else "-".join("%s%s" % (k[0], v[k]) for k in v if k != "kernel"))
def test_every_instantiation(device, name, layout, kw):
    K, N = 640, 384
    for M in sorted({1, 3, kw.get("m_block", 16), 11}):
        A, W = _case(M, N, K, layout, 7 + M)
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
        # the [K,N] MFMA kernel is built for 4 and 8 waves only
        for waves, splitk in (((4, 1), (8, 1), (4, 3), (8, 2)) if name == "kn_mfma" else ((4, 1), (2, 1), (1, 1), (4, 3), (2, 2))):
            got, _ = _run(A, W, layout, device, plan=make_plan(waves=waves, splitk=splitk, **kw))
            assert_close_f16(got, ref, "%s M=%d waves=%d S=%d" % (name, M, waves, splitk))


@pytest.mark.parametrize("unroll", [1, 2, 128])
@pytest.mark.parametrize("waves", [1, 2, 4, 8])
@pytest.mark.parametrize("splitk,fused", [(1, 0), (2, 0), (3, 1)])
def test_row_load_mfma_kernel(device, waves, splitk, fused, unroll):
    # unroll 1 / 2: 256- / 512-byte bands through the `unroll` field; 128: the `band` field
    band = 0
    if unroll == 128:
        unroll, band = 1, 128
    if waves == 8 and unroll != 1:
        pytest.skip("8-wave workgroups exist for 128- and 256-byte bands only")
    # K = 128 (half a band), 384 (one and a half), 2048 (8 bands: the unmasked path when they divide
    # evenly over waves x splits), 4480 (ragged); M <= 8 uses the 8-row A strip, M = 19 two block rows
    N = 384
    for K in (128, 384, 2048, 4480):
        for M in (1, 5, 8, 9, 16, 19):
            A, W = _case(M, N, K, NK, 70 + M + K)
            ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
            C0 = normal((M, N), gen(71), 2.0)
            refa, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK, C=C0.numpy(), accumulate=True)
            tile = 32 if (M + K // 128) % 2 else 16
            kw = dict(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=waves, splitk=splitk, fused=fused, unroll=unroll, band=band)
            got, p = _run(A, W, NK, device, plan=make_plan(**kw))
            assert p.tile_n == tile and p.grid_x == N // tile and p.block == 64 * waves
            assert p.band == (band or 256 * unroll)
            assert_close_f16(got, ref, "mfma_r M=%d K=%d" % (M, K))
            got, _ = _run(A, W, NK, device, accumulate=True, C0=C0, plan=make_plan(**kw))
            assert_close_f16(got, refa, "mfma_r accumulate M=%d K=%d" % (M, K))
    # exact small integers: any operand-layout mistake in the LDS round trip changes the bits
    g = gen(72)
    for M in (8, 16):
        A = torch.randint(-2, 3, (M, 768), generator=g).half()
        W = torch.randint(-3, 4, (N, 768), generator=g).half()
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
        for tile in (16, 32):
            got, _ = _run(A, W, NK, device, plan=make_plan(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=waves, splitk=splitk, fused=fused, unroll=unroll, band=band))
            assert (got == ref).all()


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("fused", [0, 1])
def test_split_k_two_pass_and_fused_agree_bitwise(device, layout, fused):
    # both completions sum the same fp32 partials in ascending split order
    M, N, K = 8, 512, 4096
    A, W = _case(M, N, K, layout, 61)
    kernel = capi.FG_KERNEL_KN_MFMA if layout == KN else capi.FG_KERNEL_NK_MFMA4
    base = dict(kernel=kernel, tile_n=16, m_block=8, unroll=2)
    ref_bits = None
    for splitk in (2, 4, 8):
        got, _ = _run(A, W, layout, device, plan=make_plan(splitk=splitk, fused=fused, **base))
        other, _ = _run(A, W, layout, device, plan=make_plan(splitk=splitk, fused=1 - fused, **base))
        assert (got.view(np.uint16) == other.view(np.uint16)).all()
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
        assert_close_f16(got, ref, "S=%d fused=%d" % (splitk, fused))


def test_workspace_counters_return_to_zero(device):
    # the arrival counters must be zero again after every call so the workspace can be reused
    from helpers import ptr, stream_ptr
    L = capi.lib()
    M, N, K = 16, 1024, 2048
    hdr = L.fg_workspace_header_bytes()
    ws = torch.full((hdr + 16 * M * N * 4,), 0xFF, dtype=torch.uint8, device=device)
    capi.check(L.fg_workspace_init(ptr(ws), ws.numel(), stream_ptr()), "init")
    for layout in (KN, NK):
        A, W = _case(M, N, K, layout, 71)
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
        Ad, Wd = A.to(device), W.to(device)
        C = torch.empty((M, N), dtype=torch.half, device=device)
        for splitk in (4, 2, 8, 4):
            capi.check(L.fg_gemm_f16(ptr(Ad), ptr(Wd), ptr(C), M, N, K, layout, 0, splitk, ptr(ws),
                                     ws.numel(), stream_ptr()), "gemm")
            torch.cuda.synchronize()
            assert int(ws[:hdr].view(torch.int32).abs().sum()) == 0
            assert_close_f16(C.cpu().numpy(), ref, "reuse S=%d" % splitk)


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 33])
def test_auto_plan_small(device, layout, M):
    for (N, K) in ((128, 128), (256, 1024), (1024, 384), (1152, 2176)):
        A, W = _case(M, N, K, layout, 100 * M + N)
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
        got, p = _run(A, W, layout, device)
        assert_close_f16(got, ref, "auto M=%d N=%d K=%d %s" % (M, N, K, p.as_dict()))


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("splitk", [0, 1, 2, 5])
def test_accumulate_protocol(device, layout, splitk):
    M, N, K = 8, 512, 1024
    A, W = _case(M, N, K, layout, 31)
    C0 = normal((M, N), gen(32), 4.0)
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout, C=C0.numpy(), accumulate=True)
    got, _ = _run(A, W, layout, device, accumulate=True, C0=C0, splitk=splitk)
    assert_close_f16(got, ref, "accumulate S=%d" % splitk)
    # overwrite must ignore what C held (NaN-filled by _run)
    ref0, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
    got0, _ = _run(A, W, layout, device, splitk=splitk)
    assert_close_f16(got0, ref0, "overwrite S=%d" % splitk)


def test_closed_forms(device):
    # ones x ones = K exactly (script/ncu-gemv-test.py:29-30 of the reference)
    for layout in (KN, NK):
        for K in (128, 1024, 2048):
            A = torch.ones((3, K), dtype=torch.half)
            W = torch.ones((K, 256) if layout == KN else (256, K), dtype=torch.half)
            got, _ = _run(A, W, layout, device)
            assert (got == K).all()
    # unit vector e_k selects row k of W[K,N] bit for bit
    K, N = 512, 384
    W = normal((K, N), gen(5), 1.0)
    for k in (0, 1, 255, 511):
        A = torch.zeros((2, K), dtype=torch.half)
        A[0, k] = 1.0
        A[1, k] = -2.0
        got, _ = _run(A, W, KN, device)
        assert (got[0].view(np.uint16) == W[k].numpy().view(np.uint16)).all()
        assert (got[1] == (-2.0 * W[k].float()).half().numpy()).all()
        got, _ = _run(A, W.t().contiguous(), NK, device)
        assert (got[0].view(np.uint16) == W[k].numpy().view(np.uint16)).all()


def test_small_integers_exact(device):
    # |a|,|w| <= 8 and K <= 256: every partial sum is an integer below 2^24, and |y| <= 2048
    # keeps the fp16 result exact, so any summation order must give the same bits.
    g = gen(77)
    for layout in (KN, NK):
        for M in (1, 4, 8, 16):
            K, N = 256, 256
            A = torch.randint(-2, 3, (M, K), generator=g).half()
            W = torch.randint(-3, 4, (K, N) if layout == KN else (N, K), generator=g).half()
            ref, raw = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
            assert np.abs(raw).max() <= 2048
            got, _ = _run(A, W, layout, device)
            assert (got == ref).all()


def test_row_of_batch_equals_single(device):
    # row m of an M-row call equals the M = 1 call on that row (script/cublas-gemv.py:30-35)
    M, N, K = 4, 512, 1024
    for layout in (KN, NK):
        A, W = _case(M, N, K, layout, 55)
        got, _ = _run(A, W, layout, device)
        for m in range(M):
            one, _ = _run(A[m:m + 1].contiguous(), W, layout, device)
            assert_close_f16(one[0], got[m], "row %d" % m)


def test_bitwise_reproducible(device):
    M, N, K = 16, 1024, 4096
    for layout in (KN, NK):
        A, W = _case(M, N, K, layout, 91)
        first, _ = _run(A, W, layout, device)
        for _ in range(3):
            again, _ = _run(A, W, layout, device)
            assert (first.view(np.uint16) == again.view(np.uint16)).all()


def test_error_codes_on_device(device):
    L = capi.lib()
    A = torch.zeros((8, 256), dtype=torch.half, device=device)
    W = torch.zeros((256, 256), dtype=torch.half, device=device)
    C = torch.zeros((8, 256), dtype=torch.half, device=device)
    from helpers import ptr, stream_ptr
    assert L.fg_gemm_f16(ptr(A), ptr(W), ptr(C), 8, 200, 256, NK, 0, 0, None, 0, stream_ptr()) == capi.FG_ERR_ALIGN128
    assert L.fg_gemm_f16(None, ptr(W), ptr(C), 8, 256, 256, NK, 0, 0, None, 0, stream_ptr()) == capi.FG_ERR_INVALID_ARG
    assert L.fg_gemm_f16(ptr(A), ptr(W), ptr(C), 8, 256, 256, NK, 0, 4, None, 0, stream_ptr()) == capi.FG_ERR_WORKSPACE
    assert L.fg_gemm_f16(ptr(A), ptr(W), ptr(C), 8, 256, 256, 7, 0, 0, None, 0, stream_ptr()) == capi.FG_ERR_INVALID_ARG


@pytest.mark.parametrize("layout", [KN, NK])
def test_split_deeper_than_k_has_idle_workgroups_that_contribute_zero(device, layout):
    # K = 128 is a single K unit of every kernel: with S = 16 most workgroups own no part of K and
    # must still publish an all-zero partial and arrive at the counter
    for M in (1, 4, 8, 16):
        A, W = _case(M, 256, 128, layout, 600 + M)
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
        got, p = _run(A, W, layout, device, splitk=16)
        assert p.splitk == 16
        assert_close_f16(got, ref, "S=16 on K=128, M=%d" % M)
        got, _ = _run(A, W, layout, device, splitk=3)
        assert_close_f16(got, ref, "S=3 on K=128, M=%d" % M)


@pytest.mark.parametrize("tile", [48, 64])
@pytest.mark.parametrize("waves", [1, 2, 4, 8])
@pytest.mark.parametrize("splitk,fused", [(1, 0), (2, 0), (3, 1)])
def test_row_load_mfma_kernel_three_and_four_column_blocks(device, tile, waves, splitk, fused):
    N = 768 if tile == 48 else 512
    for K in (128, 384, 2048, 4480):
        for M in (1, 5, 8, 9, 16, 19):
            A, W = _case(M, N, K, NK, 90 + M + K)
            ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
            kw = dict(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=waves, splitk=splitk, fused=fused, band=128)
            got, p = _run(A, W, NK, device, plan=make_plan(**kw))
            assert p.tile_n == tile and p.grid_x == N // tile and p.band == 128
            assert_close_f16(got, ref, "mfma_r tile %d M=%d K=%d" % (tile, M, K))
    g = gen(92)
    A = torch.randint(-2, 3, (16, 768), generator=g).half()
    W = torch.randint(-3, 4, (N, 768), generator=g).half()
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
    got, _ = _run(A, W, NK, device, plan=make_plan(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=waves, splitk=splitk, fused=fused, band=128))
    assert (got == ref).all()
    # wider tiles exist on 128-byte bands only
    with pytest.raises(capi.FastgateError):
        _run(A, W, NK, device, plan=make_plan(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=4, band=256))


@pytest.mark.parametrize("M", [8, 16])
def test_planner_takes_48_column_tiles_at_n_12288(device, M):
    N, K = 12288, 384
    assert capi.plan(M, N, K, NK, 0).tile_n == 48
    A, W = _case(M, N, K, NK, 95 + M)
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
    got, p = _run(A, W, NK, device)
    assert p.tile_n == 48 and p.band == 128 and p.grid_x == 256
    assert_close_f16(got, ref, "N=12288 M=%d" % M)


@pytest.mark.parametrize("N,tile", [(384, 24), (640, 40), (1408, 44), (2176, 34), (640, 20), (1408, 22)])
def test_row_load_mfma_kernel_tiles_that_are_not_multiples_of_16(device, N, tile):
    # a partly filled last column block: the spare rows are never loaded and never stored
    for K in (128, 384, 2048, 4480):
        for M in (1, 5, 8, 9, 16, 19):
            A, W = _case(M, N, K, NK, 97 + M + K)
            ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
            got, p = _run(A, W, NK, device, plan=make_plan(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=8, band=128))
            assert p.tile_n == tile and p.grid_x == N // tile and p.grid_z == 1
            assert_close_f16(got, ref, "mfma_r tile %d M=%d K=%d" % (tile, M, K))
            C0 = normal((M, N), gen(98), 2.0)
            refa, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK, C=C0.numpy(), accumulate=True)
            got, _ = _run(A, W, NK, device, accumulate=True, C0=C0, plan=make_plan(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=8, band=128))
            assert_close_f16(got, refa, "mfma_r tile %d accumulate M=%d K=%d" % (tile, M, K))
    g = gen(99)
    A = torch.randint(-2, 3, (16, 768), generator=g).half()
    W = torch.randint(-3, 4, (N, 768), generator=g).half()
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
    got, _ = _run(A, W, NK, device, plan=make_plan(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=8, band=128))
    assert (got == ref).all()
    # such tiles exist without split-K and with eight waves only
    for bad in (dict(splitk=2), dict(waves=4)):
        kw = dict(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, waves=8, band=128)
        kw.update(bad)
        with pytest.raises(capi.FastgateError):
            _run(A, W, NK, device, plan=make_plan(**kw))


def test_planner_gives_each_cu_n_over_256_columns_at_n_11008(device):
    N, K, M = 11008, 1152, 16
    A, W = _case(M, N, K, NK, 101)
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
    got, p = _run(A, W, NK, device)
    assert p.tile_n == 43 and p.grid_x == 256 and p.band == 128 and p.waves == 8
    assert_close_f16(got, ref, "N=11008 M=16")


def test_in_launch_split_k_is_stable_over_many_back_to_back_calls(device):
    # 600 calls that complete split-K inside the launch, alternating shapes and layouts on ONE
    # workspace with no host synchronisation in between: every output must equal the first
    # output of its shape bit for bit, and the counters must end at zero
    from helpers import ptr, stream_ptr
    L = capi.lib()
    hdr = L.fg_workspace_header_bytes()
    ws = torch.full((hdr + 16 * 16 * 4096 * 4,), 0xFF, dtype=torch.uint8, device=device)
    capi.check(L.fg_workspace_init(ptr(ws), ws.numel(), stream_ptr()), "init")
    cases = []
    for i, (M, N, K, layout, S) in enumerate([(1, 4096, 4096, KN, 8), (8, 2048, 4096, KN, 5), (16, 1024, 8192, KN, 3),
                                              (16, 3072, 6144, NK, 4), (5, 4096, 2048, KN, 16), (12, 1024, 8192, NK, 4)]):
        A, W = _case(M, N, K, layout, 500 + i)
        Ad, Wd = A.to(device), W.to(device)
        p = capi.plan(M, N, K, layout, S)
        assert p.splitk == S and p.fused in (1, 2), p.as_dict()
        outs = [torch.full((M, N), float("nan"), dtype=torch.half, device=device) for _ in range(100)]
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
        cases.append((M, N, K, layout, S, Ad, Wd, outs, ref))
    for it in range(100):
        for (M, N, K, layout, S, Ad, Wd, outs, _) in cases:
            st = L.fg_gemm_f16(ptr(Ad), ptr(Wd), ptr(outs[it]), M, N, K, layout, 0, S, ptr(ws), ws.numel(), stream_ptr())
            assert st == 0
    torch.cuda.synchronize()
    assert int(ws[:hdr].view(torch.int32).abs().sum()) == 0
    for (M, N, K, layout, S, Ad, Wd, outs, ref) in cases:
        first = outs[0].cpu().numpy()
        assert_close_f16(first, ref, "M=%d N=%d K=%d S=%d" % (M, N, K, S))
        stack = torch.stack(outs).view(torch.int16)
        assert bool((stack == stack[0]).all()), (M, N, K, layout, S)


@pytest.mark.parametrize("layout", [KN, NK])
def test_without_a_workspace_the_library_runs_unsplit(device, layout):
    # the planner would split these shapes; with no workspace (or too small a one) the call must
    # still give the right result, and a forced split must still be refused
    from helpers import ptr, stream_ptr
    L = capi.lib()
    M, N, K = 8, 1024, 4096
    assert layout == NK or capi.plan(M, N, K, layout, 0).splitk > 1
    A, W = _case(M, N, K, layout, 610)
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), layout)
    Ad, Wd = A.to(device), W.to(device)
    C = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
    assert L.fg_gemm_f16(ptr(Ad), ptr(Wd), ptr(C), M, N, K, layout, 0, 0, None, 0, stream_ptr()) == capi.FG_OK
    torch.cuda.synchronize()
    assert_close_f16(C.cpu().numpy(), ref, "no workspace")
    small = torch.zeros(1024, dtype=torch.uint8, device=device)
    C.fill_(float("nan"))
    assert L.fg_gemm_f16(ptr(Ad), ptr(Wd), ptr(C), M, N, K, layout, 0, 0, ptr(small), small.numel(), stream_ptr()) == capi.FG_OK
    torch.cuda.synchronize()
    assert_close_f16(C.cpu().numpy(), ref, "workspace too small")
    assert L.fg_gemm_f16(ptr(Ad), ptr(Wd), ptr(C), M, N, K, layout, 0, 4, None, 0, stream_ptr()) == capi.FG_ERR_WORKSPACE


@pytest.mark.parametrize("tile", [16, 32, 48])
@pytest.mark.parametrize("waves", [2, 4, 8])
@pytest.mark.parametrize("splitk,fused", [(1, 0), (2, 0), (3, 1)])
def test_row_load_mfma_kernel_with_32_row_blocks(device, tile, waves, splitk, fused):
    # two MFMA row blocks per workgroup: 17..32 rows read the weights once; more rows add block rows
    N = 768 if tile == 48 else 384
    for K in (128, 384, 2048, 4480):
        for M in (17, 24, 31, 32, 33, 47, 64):
            A, W = _case(M, N, K, NK, 110 + M + K)
            ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
            kw = dict(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, m_block=32, waves=waves, splitk=splitk, fused=fused, band=128)
            got, p = _run(A, W, NK, device, plan=make_plan(**kw))
            assert p.m_block == 32 and p.grid_y == -(-M // 32) and p.tile_n == tile
            assert_close_f16(got, ref, "mfma_r 32-row blocks tile %d M=%d K=%d" % (tile, M, K))
    g = gen(111)
    A = torch.randint(-2, 3, (32, 768), generator=g).half()
    W = torch.randint(-3, 4, (N, 768), generator=g).half()
    ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
    got, _ = _run(A, W, NK, device, plan=make_plan(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, m_block=32, waves=waves, splitk=splitk, fused=fused, band=128))
    assert (got == ref).all()
    C0 = normal((32, N), gen(112), 2.0)
    refa, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK, C=C0.numpy(), accumulate=True)
    got, _ = _run(A, W, NK, device, accumulate=True, C0=C0, plan=make_plan(kernel=capi.FG_KERNEL_NK_MFMA_R, tile_n=tile, m_block=32, waves=waves, splitk=splitk, fused=fused, band=128))
    assert_close_f16(got, refa, "32-row blocks, accumulate")


@pytest.mark.parametrize("M", [17, 32, 40])
def test_planner_uses_32_row_blocks_beyond_16_rows(device, M):
    for (N, K) in ((1024, 2048), (8192, 256), (12288, 384)):
        p = capi.plan(M, N, K, NK, 0)
        assert p.kernel == capi.FG_KERNEL_NK_MFMA_R and p.m_block == 32 and p.band == 128, p.as_dict()
        A, W = _case(M, N, K, NK, 120 + M)
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), NK)
        got, _ = _run(A, W, NK, device)
        assert_close_f16(got, ref, "auto plan M=%d N=%d K=%d" % (M, N, K))


@pytest.mark.parametrize("M", [1, 8, 16])
def test_planner_splits_narrow_kn_outputs(device, M):
    # sixteen [K,N] tiles or fewer: deep splits that complete through atomics, or for nine rows and more
    # through flags in one L2 (the pinned factors are in tests/test_host.py) -- each checked against the
    # oracle through the library's plan
    for (N, K) in ((2048, 4096), (2048, 8192), (1024, 16384), (2048, 16384), (1024, 11008)):
        p = capi.plan(M, N, K, KN, 0)
        assert p.splitk >= 12 and p.fused in (2, 3), p.as_dict()
        A, W = _case(M, N, K, KN, 140 + M)
        ref, _ = oracle.gemm_f16(A.numpy(), W.numpy(), KN)
        got, _ = _run(A, W, KN, device)
        assert_close_f16(got, ref, "auto plan M=%d N=%d K=%d" % (M, N, K))


@pytest.mark.parametrize("M,N,K,layout,want", [
    # [K,N], flags in one L2: (split, waves, units a step)
    (8, 9216, 4096, KN, (7, 4, 1)), (16, 18432, 2048, KN, (5, 4, 1)), (5, 22016, 4096, KN, (4, 4, 1)),
    (16, 12800, 4096, KN, (7, 4, 1)), (4, 20480, 4096, KN, (6, 4, 2)), (16, 24576, 4096, KN, (4, 4, 1)),
    (16, 2560, 4096, KN, (8, 8, 1)), (16, 3584, 3072, KN, (8, 4, 1)), (8, 6144, 4096, KN, (9, 4, 1)),
    (16, 10240, 3072, KN, (6, 4, 1)), (16, 5120, 8192, KN, (6, 4, 1)), (8, 12288, 2048, KN, (8, 4, 1)),
    (3, 8192, 3072, KN, (8, 4, 1)),
    # [K,N], one or two rows, atomics
    (1, 6144, 4096, KN, (16, 4, 2)), (2, 18432, 4096, KN, (7, 4, 1)), (1, 22016, 4096, KN, (4, 4, 2)),
    (2, 4096, 4096, KN, (16, 4, 1)),
    # [N,K]: (tile, split, band)
    (16, 2560, 8192, NK, (32, 3, 128)), (8, 12800, 4096, NK, (64, 1, 128)), (16, 13056, 4096, NK, (64, 1, 128)),
])
def test_plans_for_widths_between_the_fitted_ones(device, M, N, K, layout, want):
    # the planner's rules by tile count: each plan runs at its real width and three windows of 128
    # output columns are held to the oracle
    A, W = _case(M, N, K, layout, 7000 + M + N // 128 + K // 128)
    got, p = _run(A, W, layout, device)
    if layout == KN:
        assert (p.splitk, p.waves, p.unroll) == want, p.as_dict()
        assert p.fused == (3 if M >= 3 else 2)
    else:
        assert (p.tile_n, p.splitk, p.band) == want, p.as_dict()
    assert not np.isnan(got.astype(np.float32)).any()
    for lo in (0, (N // 2) // 128 * 128, N - 128):
        Wwin = W[:, lo:lo + 128] if layout == KN else W[lo:lo + 128]
        ref, _ = oracle.gemm_f16(A.numpy(), Wwin.contiguous().numpy(), layout)
        assert_close_f16(got[:, lo:lo + 128], ref, "columns %d.." % lo)
