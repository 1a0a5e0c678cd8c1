"""The pybind11 operator surface on the GPU: every reference name, with the reference's
argument order and C protocol, against the oracle's restatement of that operator."""
import zlib

import numpy as np
import pytest
import torch

import oracle
from helpers import assert_close_f16, gen, normal, uniform_pm1

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sg():
    import fastgate_amd

    return fastgate_amd.speedgate


@pytest.mark.parametrize("name", sorted(oracle.GEMM_OPS))
def test_gemm_operator_semantics(device, sg, name):
    layout, protocol, has_bz = oracle.GEMM_OPS[name]
    g = gen(zlib.crc32(name.encode()) % 10000)
    for M in (1, 8, 16):
        K, N = 1024, 768
        A = normal((M, K), g)
        B = normal((K, N) if layout == oracle.W_KN else (N, K), g, 0.02)
        C0 = normal((M, N), g, 2.0)  # what the caller left in C
        for bz in ((2, 8, 0) if has_bz else (None,)):
            Cd = C0.to(device).clone()
            args = (A.to(device), B.to(device), Cd) + ((bz,) if has_bz else ())
            assert getattr(sg, name)(*args) is None
            torch.cuda.synchronize()
            ref = oracle.gemm_op(name, A.numpy(), B.numpy(), C0.numpy(), bz=bz)
            assert_close_f16(Cd.cpu().numpy(), ref, "%s M=%d bz=%s (%s)" % (name, M, bz, protocol))


def test_legacy_edgemm_names(device, sg):
    g = gen(12)
    A, B = normal((8, 512), g), normal((512, 256), g, 0.02)
    ref, _ = oracle.gemm_f16(A.numpy(), B.numpy(), oracle.W_KN)
    for name in ("edgemm", "edgemm_m8n256k64", "edgemm_m8n128k64", "edgemm_m8n128k128"):
        C = torch.full((8, 256), float("nan"), dtype=torch.half, device=device)
        getattr(sg, name)(A.to(device), B.to(device), C)
        assert_close_f16(C.cpu().numpy(), ref, name)
    C0 = normal((1, 256), g)
    refa, _ = oracle.gemm_f16(A[:1].numpy(), B.numpy(), oracle.W_KN, C=C0.numpy(), accumulate=True)
    for name in ("edgemv_m1n128k64x4", "edgemv_m1n256k64x4"):
        C = C0.to(device).clone()
        getattr(sg, name)(A[:1].contiguous().to(device), B.to(device), C)
        assert_close_f16(C.cpu().numpy(), refa, name)


def test_fastgemv_weight_first_and_shapes(device, sg):
    g = gen(1001)
    N, K = 1024, 2048
    W = uniform_pm1((N, K), g)
    x = uniform_pm1((1, K), g)
    ref = oracle.fastgemv(W.numpy(), x.numpy())
    Wd = W.to(device)
    for xs, ys in (((1, K), (N,)), ((K, 1), (N, 1)), ((K,), (1, N))):
        y = torch.full(ys, float("nan"), dtype=torch.half, device=device)
        sg.fastgemv(Wd, x.reshape(xs).contiguous().to(device), y)
        assert_close_f16(y.cpu().numpy().reshape(-1), ref, "fastgemv %s" % (xs,))
        y.fill_(float("nan"))
        sg.fastgemv_tuned(Wd, x.reshape(xs).contiguous().to(device), y)
        assert_close_f16(y.cpu().numpy().reshape(-1), ref, "fastgemv_tuned %s" % (xs,))
    # ones x ones = K (script/ncu-gemv-test.py:29-30)
    y = torch.zeros(N, dtype=torch.half, device=device)
    sg.fastgemv(torch.ones((N, K), dtype=torch.half, device=device),
                torch.ones((1, K), dtype=torch.half, device=device), y)
    assert (y.cpu() == K).all()


@pytest.mark.parametrize("M", [1, 2, 5, 8])
def test_fastgemv_extend_and_fastgemm(device, sg, M):
    g = gen(1100 + M)
    N, K = 512, 1024
    W, X = normal((N, K), g, 0.05), normal((M, K), g)
    ref = oracle.fastgemv_extend(W.numpy(), X.numpy())
    for fn in (sg.fastgemv_extend, sg.fastgemm):
        C = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
        fn(W.to(device), X.to(device), C)
        assert_close_f16(C.cpu().numpy(), ref, fn.__name__)


def test_fastgemv_int8_defaults_and_extension(device, sg):
    g = gen(1004)
    N, K = 1024, 2048
    x = (normal((1, K), g) * 0.05).half()
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    y = torch.empty(N, dtype=torch.half, device=device)
    sg.fastgemv_int8(Wq.to(device), x.to(device), y)
    assert_close_f16(y.cpu().numpy(), oracle.fastgemv_int8(Wq.numpy(), x.numpy()), "defaults")
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    x1 = normal((1, K), g)
    sg.fastgemv_int8(Wq.to(device), x1.to(device), y, scale=scale.to(device))
    ref, _ = oracle.gemv_w8a16(Wq.numpy(), x1.numpy(), scale.numpy())
    assert_close_f16(y.cpu().numpy(), ref.reshape(-1), "per-channel scale")


def test_fastgemv_int8_takes_up_to_16_activation_rows(device, sg):
    g = gen(1014)
    N, K = 1024, 1152
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    scale = (torch.rand(N, generator=g) * 0.009 + 0.001).half()
    for M in (2, 7, 16):
        x = normal((M, K), g)
        y = torch.full((M, N), float("nan"), dtype=torch.half, device=device)
        sg.fastgemv_int8(Wq.to(device), x.to(device), y, scale=scale.to(device))
        ref, _ = oracle.gemv_w8a16(Wq.numpy(), x.numpy(), scale.numpy())
        assert_close_f16(y.cpu().numpy(), ref, "M=%d" % M)
    x = normal((17, K), g)
    y = torch.empty((17, N), dtype=torch.half, device=device)
    with pytest.raises(RuntimeError, match="at most 16 activation rows"):
        sg.fastgemv_int8(Wq.to(device), x.to(device), y)


def test_integer_ops(device, sg):
    g = gen(1005)
    N, K = 512, 1024
    Wq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    xq = torch.randint(-128, 128, (1, K), generator=g, dtype=torch.int8)
    acc = torch.empty((1, N), dtype=torch.int32, device=device)
    sg.gemv_i8i8_i32(Wq.to(device), xq.to(device), acc)
    assert (acc.cpu().numpy() == oracle.gemv_i8i8_i32(Wq.numpy(), xq.numpy())).all()


def test_vendor_comparators(device, sg):
    g = gen(9)
    A, B = normal((16, 512), g), normal((512, 256), g, 0.02)
    ref, _ = oracle.gemm_f16(A.numpy(), B.numpy(), oracle.W_KN)
    C = torch.empty((16, 256), dtype=torch.half, device=device)
    sg.hgemm(A.to(device), B.to(device), C)
    assert_close_f16(C.cpu().numpy(), ref, "hgemm")
    for fn in (sg.hgemm_tr, sg.mma):
        C.zero_()
        fn(A.to(device), B.t().contiguous().to(device), C)
        assert_close_f16(C.cpu().numpy(), ref, fn.__name__)


def test_errors_on_device(device, sg):
    h = dict(dtype=torch.half, device=device)
    A, B, C = torch.zeros((8, 256), **h), torch.zeros((256, 384), **h), torch.zeros((8, 384), **h)
    with pytest.raises(ValueError, match="multiple of 128"):
        sg.edgemm_m8n128k64x4(torch.zeros((8, 200), **h), torch.zeros((200, 384), **h), C)
    with pytest.raises(ValueError, match="multiple of 128"):
        sg.edgemm_m8n128k64x4_bt(A, torch.zeros((100, 256), **h), C)
    with pytest.raises(RuntimeError, match="inner dimensions"):
        sg.edgemm_m8n128k64x4(A, torch.zeros((384, 384), **h), C)
    with pytest.raises(RuntimeError, match="Half"):
        sg.edgemm_m8n128k64x4(A.float(), B, C)
    with pytest.raises(RuntimeError, match="contiguous"):
        sg.edgemm_m8n128k64x4(A, torch.zeros((384, 256), **h).t(), C)
    with pytest.raises(RuntimeError, match="M\\*N"):
        sg.edgemm_m8n128k64x4(A, B, torch.zeros((8, 128), **h))
    with pytest.raises(RuntimeError, match="HIP device"):
        sg.edgemm_m8n128k64x4(A.cpu(), B, C)


def test_runs_on_the_current_stream(device, sg):
    g = gen(3)
    A, B = normal((8, 1024), g).to(device), normal((1024, 1024), g, 0.02).to(device)
    ref, _ = oracle.gemm_f16(A.cpu().numpy(), B.cpu().numpy(), oracle.W_KN)
    s = torch.cuda.Stream()
    C = torch.zeros((8, 1024), dtype=torch.half, device=device)
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        for _ in range(3):
            sg.edgemm_m8n128k64x4(A, B, C)
    s.synchronize()
    assert_close_f16(C.cpu().numpy(), ref, "side stream")


def test_reference_harness_flow(device):
    # the reference's table row (script/standard-test.py): torch, vendor, then each operator with
    # its time, share of outputs within 100 and the allclose verdict
    import eed.backend as backend
    from fastgate_amd import harness
    funcs = [backend.edgemm_m8n128k64x4, backend.edgemm_m8n128k64x4_bt, backend.gemm_m8n64k128x8_bt_exp,
             backend.flat_gemm_m8n256k64x8, backend.edgemm_m8n64k128x8_bt_tuning]
    row = harness.run_config(funcs, 8, 1024, 2048, warmup=2, iters=3, bz=2)
    assert set(row["ops"]) == {"edgemm_m8n128k64x4", "edgemm_m8n128k64x4_bt", "gemm_m8n64k128x8_bt_exp",
                                "flat_gemm_m8n256k64x8"}   # the alias shares its target's name
    for name, e in row["ops"].items():
        assert e["share_within_100"] == 1.0 and e["allclose"], (name, e)
        assert e["ms"] > 0
    assert row["vendor_share_within_100"] == 1.0
    assert len(harness.format_row(row).split()) == 3 + 2 + len(row["ops"]) + 1 + len(row["ops"])
    # the GEMV family: weight first
    row = harness.run_config([backend.fastgemv, backend.fastgemv_tuned], 1, 2048, 1024, warmup=1, iters=2)
    assert all(e["allclose"] for e in row["ops"].values())


def test_reference_iter_func_flow(device):
    # script/standard-test.py:190-250: each operator twice on fresh outputs, run against run (here
    # bit for bit), run against torch.matmul, then the timing loops
    import eed.backend as backend
    from fastgate_amd import harness
    funcs = [backend.edgemm_m8n128k64x4, backend.edgemm_m8n128k64x4_bt, backend.flat_gemm_m8n256k32x16,
             backend.gemm_m8n64k128x8_bt_exp, backend.fastgemv_extend]
    rows = harness.iter_func(funcs, [(8, 1024, 2048), (1, 4096, 1024), (16, 2048, 1152)], warmup=1, iters=2)
    assert len(rows) == len(funcs) * 3
    for e in rows:
        assert e["runs_allclose"] and e["runs_bitwise_equal"] and e["allclose_to_torch"], e
        assert e["ms"] > 0 and e["torch_ms"] > 0


def test_operators_replay_correctly_from_a_hip_graph(device):
    # serving loops capture the calls once and replay them: every launch (split-K second pass and
    # in-launch completion included) must be capturable and give the eager result on each replay
    import fastgate_amd
    sg = fastgate_amd.speedgate
    g = gen(4242)
    K, N = 2048, 1024
    Wkn = normal((K, N), g, 0.05).to(device)
    Wnk = Wkn.t().contiguous()
    Wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).to(device)
    acts = {M: normal((M, K), g, 1.0).to(device) for M in (1, 8, 16)}
    outs = {k: torch.zeros((M, N), dtype=torch.half, device=device)
            for k, M in (("kn1", 1), ("kn8", 8), ("kn16", 16), ("nk8", 8), ("nk16", 16), ("gemv", 1), ("i8", 1))}

    def step():
        sg.edgemm_m8n128k64x4(acts[1], Wkn, outs["kn1"])
        sg.edgemm_m8n128k64x4(acts[8], Wkn, outs["kn8"])
        sg.edgemm_m8n128k64x4(acts[16], Wkn, outs["kn16"])
        sg.edgemm_m8n128k64x4_bt(acts[8], Wnk, outs["nk8"])
        sg.edgemm_m8n128k64x4_bt(acts[16], Wnk, outs["nk16"])
        sg.fastgemv(Wnk, acts[1], outs["gemv"])
        sg.fastgemv_int8(Wq, acts[1], outs["i8"])

    step()                      # eager: also sizes the cached workspace outside the capture
    torch.cuda.synchronize()
    want = {k: v.clone() for k, v in outs.items()}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                  # the capture stream gets its own workspace first
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.synchronize()
    for replay in range(3):
        for v in outs.values():
            v.fill_(float("nan"))
        # eager work of the program between replays
        sg.edgemm_m8n128k64x4(acts[8], Wkn, torch.empty((8, N), dtype=torch.half, device=device))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k in outs:
            assert torch.equal(outs[k], want[k]), (replay, k)


@pytest.mark.parametrize("args", [
    ["--m", "1", "--n", "4096", "--k", "4096", "--layout", "nk"],
    ["--m", "8", "--n", "2048", "--k", "4480", "--layout", "kn"],
    ["--m", "16", "--n", "1024", "--k", "8192", "--layout", "kn"],
    ["--m", "16", "--n", "3072", "--k", "1152", "--layout", "nk"],
    ["--m", "3", "--n", "1024", "--k", "2048", "--dtype", "i8"],
    ["--m", "1", "--n", "1024", "--k", "2048", "--dtype", "i8"],
    ["--m", "1", "--n", "1024", "--k", "4096", "--dtype", "i4"],
    ["--m", "4", "--n", "1024", "--k", "1152", "--dtype", "i4"],
], ids=lambda a: "-".join(x.lstrip("-") for x in a))
def test_standalone_cpp_caller_of_the_c_abi(device, args):
    """fg_cbench: hipMalloc + include/fastgate.h only (no torch in that process); it checks a closed
    form on the device result and reports a timing."""
    import json
    import subprocess
    from pathlib import Path

    exe = Path(__file__).resolve().parent.parent / "fastgate_amd" / "fg_cbench"
    assert exe.exists(), "fastgate_amd/fg_cbench is not built (python -m fastgate_amd.build)"
    out = subprocess.run([str(exe), *args, "--iters", "20"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    assert rec["ok"] is True and rec["mismatches"] == 0 and rec["us_per_call"] > 0


def test_two_streams_with_split_k_calls_in_flight_do_not_interfere(device, sg):
    # the binding keeps one split-K workspace per (device, stream): calls that overlap in time on
    # different streams must each complete their own tiles
    g = gen(77)
    K, N = 4096, 1024                        # [K,N] at this size always splits K
    assert sg.plan(8, N, K, sg.W_KN)["splitk"] > 1
    W = [normal((K, N), g, 0.03).to(device) for _ in range(2)]
    A = [normal((8, K), g).to(device) for _ in range(2)]
    ref = [oracle.gemm_f16(A[i].cpu().numpy(), W[i].cpu().numpy(), oracle.W_KN)[0] for i in range(2)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[torch.full((8, N), float("nan"), dtype=torch.half, device=device) for _ in range(30)] for _ in range(2)]
    torch.cuda.synchronize()
    for it in range(30):
        for i in range(2):
            with torch.cuda.stream(streams[i]):
                sg.edgemm_m8n128k64x4(A[i], W[i], outs[i][it])
    torch.cuda.synchronize()
    for i in range(2):
        first = outs[i][0].cpu().numpy()
        assert_close_f16(first, ref[i], "stream %d" % i)
        for it in range(1, 30):
            assert (outs[i][it].cpu().numpy().view(np.uint16) == first.view(np.uint16)).all(), (i, it)


@pytest.mark.gpu
@pytest.mark.parametrize("completion", ["two-pass", "counter", "atomic"])
def test_completion_switch_end_to_end(completion):
    """FASTGATE_SPLITK_COMPLETION is read once per process: a child process with the variable set
    runs split [K,N] and [N,K] products through the binding and compares them with torch.matmul."""
    import os
    import subprocess
    import sys
    from pathlib import Path
    code = r'''
import torch
from fastgate_amd import capi, speedgate as sg
want = {"two-pass": 0, "counter": 1, "atomic": 2}[%r]
torch.manual_seed(3)
for (M, N, K, op, layout) in ((8, 4096, 4096, "edgemm_m8n128k64x4", 0), (1, 2048, 8192, "edgemm_m8n128k64x4", 0),
                              (16, 2048, 8192, "edgemm_m8n128k64x4_bt", 1)):
    p = capi.plan(M, N, K, layout)
    assert p.splitk > 1 and p.fused == want, (M, N, K, p.as_dict())
    A = torch.randn(M, K, device="cuda").half()
    W = (torch.randn((K, N) if layout == 0 else (N, K), device="cuda") * 0.05).half()
    C = torch.empty(M, N, dtype=torch.half, device="cuda")
    getattr(sg, op)(A, W, C)
    ref = A.float() @ (W.float() if layout == 0 else W.float().t())
    assert bool(((C.float() - ref).abs() <= 1e-2 + 2e-3 * ref.abs()).all()), (M, N, K)
print("ok")
''' % completion
    root = Path(__file__).resolve().parent.parent
    env = dict(os.environ, FASTGATE_SPLITK_COMPLETION=completion)
    out = subprocess.run([sys.executable, "-c", code], env=env, cwd=root, capture_output=True, text=True, timeout=110)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr
