"""The reference's test-and-time flow (script/standard-test.py) for the MI355X operators.

What is kept, with the line of the reference it follows:
  * inputs: A ~ N(0,1), B ~ N(1,1) with columns -4:-2 divided by 100, fp16 (:140-142);
  * three calling conventions (:89-118): "all transposed" ops take (B_t, A_t, C_t) -- the
    weight-first GEMV family; "B transposed" ops take (A, B_t, C); the rest take (A, B, C);
    ops with a trailing split factor get it appended;
  * timing (:125-137): `warmup` untimed calls, then `iters` calls each bracketed by a device
    synchronize and a host clock; the figure is the mean in milliseconds per call;
  * verdicts: the share of outputs within 100 of torch.matmul (:152-166) and
    torch.allclose(rtol=1e-1, atol=1e-2) (:236);
  * the per-operator check of `iter_func` (:190-250): inputs uniform in [0, 1), the operator called
    twice on fresh outputs, the two runs compared, the first compared with torch.matmul, then
    torch and the operator timed with the same loop.
The vendor column (`hgemm`, cuBLAS in the reference) is this library's `hgemm`, i.e. hipBLASLt
through ATen.  Nothing here computes on the CPU.
"""
from __future__ import annotations

import time

import torch

WARMUP = 10   # script/standard-test.py:120
ITERS = 100   # script/standard-test.py:121

# Calling conventions by operator name.
ALL_TRANSPOSED = ("fastgemv", "fastgemv_tuned", "fastgemv_extend", "fastgemm")
B_TRANSPOSED = ("edgemm_m8n128k64x4_bt", "edgemm_m8n128k64x4_tr_amd", "gemm_m8n128k64x4_bt",
                "gemm_m8n32k128x8_bt", "gemm_m8n64k128x8_bt_exp", "gemm_m8n32k256x8_bt",
                "gemm_m8n32k256x8_bt_bz2", "hgemm_tr", "mma",
                "edgemm_m8n32k128x8_bt", "edgemm_m8n32k256x8_bt",
                "edgemm_m8n64k128x8_bt_tuning", "edgemm_m8n32k256x8_bt_tuning")
TAKES_BZ = ("flat_gemm_m8n128k64x4_bz1", "flat_gemm_m8n256k64x8", "flat_gemm_m8n512k32x16",
            "flat_gemm_m8n64k128x8", "flat_gemm_m8n32k256x8", "gemm_m8n64k128x8_bt_exp",
            "gemm_m8n32k256x8_bt_bz2", "edgemm_m8n64k128x8_bt_tuning", "edgemm_m8n32k256x8_bt_tuning")


def _name(func) -> str:
    return getattr(func, "__name__", type(func).__name__)


def make_inputs(M: int, K: int, N: int, device="cuda", seed: int = 10):
    """A, B, B_t and zeroed outputs as script/standard-test.py:140-149 builds them."""
    g = torch.Generator(device=device).manual_seed(seed)
    A = torch.empty((M, K), dtype=torch.float16, device=device).normal_(mean=0.0, std=1.0, generator=g)
    B = torch.empty((K, N), dtype=torch.float16, device=device).normal_(mean=1.0, std=1.0, generator=g)
    B[:, -4:-2] = B[:, -4:-2] / 100
    return A, B, B.transpose(0, 1).contiguous()


def dispatch_func(func, A, B, C, A_T, B_T, C_T):
    """script/standard-test.py:89-97: operands in their natural layouts, transposed copies at hand."""
    name = _name(func)
    if name in ALL_TRANSPOSED:
        func(B_T, A_T, C_T)
    elif name in B_TRANSPOSED:
        func(A, B_T, C)
    elif isinstance(func, torch.nn.Linear):
        C.copy_(func(A))
    else:
        func(A, B, C)


def dispatch_func_btrans(func, A, B_T, C, bz: int = 1):
    """script/standard-test.py:100-118: A is [M,K], the weight is given transposed ([N,K])."""
    name = _name(func)
    if name in ALL_TRANSPOSED:
        # weight-first GEMV family: (mat[N,K], vec[M,K], res[M,N])
        func(B_T, A, C)
    elif name in TAKES_BZ and name in B_TRANSPOSED:
        func(A, B_T, C, bz)
    elif name in B_TRANSPOSED:
        func(A, B_T, C)
    elif isinstance(func, torch.nn.Linear):
        C.copy_(func(A))
    elif name in TAKES_BZ:
        func(A, B_T.transpose(0, 1).contiguous(), C, bz)
    else:
        func(A, B_T.transpose(0, 1).contiguous(), C)


def speed_test(call, warmup: int = WARMUP, iters: int = ITERS) -> float:
    """Mean milliseconds per call, each call bracketed by synchronizes (script/standard-test.py:125-137)."""
    for _ in range(warmup):
        call()
    total = 0.0
    for _ in range(iters):
        torch.cuda.synchronize()
        st = time.time()
        call()
        torch.cuda.synchronize()
        total += time.time() - st
    return total * 1e3 / iters


def share_within(C_ref, C, bound: float = 100.0) -> float:
    """Share of outputs with |C_ref - C| <= bound (script/standard-test.py:152)."""
    return float((C_ref.float() - C.float()).abs().le(bound).float().mean())


def run_config(funcs, M: int, K: int, N: int, warmup: int = WARMUP, iters: int = ITERS, bz: int = 1,
               device="cuda"):
    """One row of the reference's table: torch and vendor times, then per operator the time, the
    share within 100 and the allclose verdict against torch.matmul."""
    import fastgate_amd
    sg = fastgate_amd.speedgate
    A, B, B_T = make_inputs(M, K, N, device)
    C_ref = torch.zeros((M, N), dtype=torch.float16, device=device)
    torch.matmul(A, B, out=C_ref)
    C_v = torch.zeros_like(C_ref)
    sg.hgemm(A, B, C_v)
    row = {"M": M, "K": K, "N": N,
           "torch_ms": speed_test(lambda: torch.matmul(A, B, out=C_ref), warmup, iters),
           "vendor_ms": speed_test(lambda: sg.hgemm(A, B, C_v), warmup, iters),
           "vendor_share_within_100": share_within(C_ref, C_v), "ops": {}}
    for f in funcs:
        C = torch.zeros((M, N), dtype=torch.float16, device=device)
        dispatch_func_btrans(f, A, B_T, C, bz)   # accumulate-type ops start from a zeroed C
        torch.cuda.synchronize()
        entry = {"share_within_100": share_within(C_ref, C),
                 "allclose": bool(torch.allclose(C_ref, C, rtol=1e-1, atol=1e-2))}
        C_t = torch.zeros_like(C)
        entry["ms"] = speed_test(lambda: dispatch_func_btrans(f, A, B_T, C_t, bz), warmup, iters)
        row["ops"][_name(f)] = entry
    return row


def iter_func(funcs, configs, warmup: int = WARMUP, iters: int = ITERS, device="cuda", seed: int = 10):
    """script/standard-test.py:190-250 for every (operator, (M, K, N)): A, B uniform in [0, 1) with
    columns -4:-2 of B divided by 100; the operator runs twice, on two zeroed outputs; the runs are
    compared with each other (allclose in the reference; here the bits are compared as well, since
    the operators are reproducible run to run) and the first with torch.matmul; then torch.matmul
    and the operator are timed.  The reference calls every operator as func(A, B, C); the calling
    convention of each name (weight first, transposed weight, trailing bz) is applied here as
    dispatch_func does.  Returns one dict per (operator, config)."""
    out = []
    for f in funcs:
        for (M, K, N) in configs:
            g = torch.Generator(device=device).manual_seed(seed)
            A = torch.rand((M, K), dtype=torch.float16, device=device, generator=g)
            B = torch.rand((K, N), dtype=torch.float16, device=device, generator=g)
            B[:, -4:-2] = B[:, -4:-2] / 100
            C_ref = torch.zeros((M, N), dtype=torch.float16, device=device)
            C = torch.zeros_like(C_ref)
            C2 = torch.zeros_like(C_ref)
            B_T = B.transpose(0, 1).contiguous()
            torch.matmul(A, B, out=C_ref)
            dispatch_func_btrans(f, A, B_T, C)
            torch.cuda.synchronize()
            dispatch_func_btrans(f, A, B_T, C2)
            torch.cuda.synchronize()
            entry = {"op": _name(f), "M": M, "K": K, "N": N,
                     "runs_allclose": bool(torch.allclose(C2, C, rtol=1e-1, atol=1e-2)),
                     "runs_bitwise_equal": bool(torch.equal(C2.view(torch.int16), C.view(torch.int16))),
                     "allclose_to_torch": bool(torch.allclose(C_ref, C, rtol=1e-1, atol=1e-2))}
            entry["torch_ms"] = speed_test(lambda: torch.matmul(A, B, out=C_ref), warmup, iters)
            C_t = torch.zeros_like(C_ref)
            entry["ms"] = speed_test(lambda: dispatch_func_btrans(f, A, B_T, C_t), warmup, iters)
            out.append(entry)
    return out


def format_row(row) -> str:
    """`M K N torch vendor ours... vendor_acc ours_acc...` as script/standard-test.py:181-187 prints."""
    ops = row["ops"]
    parts = ["%d %d %d" % (row["M"], row["K"], row["N"]), "%.4f" % row["torch_ms"], "%.4f" % row["vendor_ms"]]
    parts += ["%.4f" % e["ms"] for e in ops.values()]
    parts += [repr(row["vendor_share_within_100"])] + [repr(e["share_within_100"]) for e in ops.values()]
    return " ".join(parts)
