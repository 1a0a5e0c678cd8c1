#!/usr/bin/env python3
"""Benchmark of the small-batch GEMM/GEMV hot path on one MI355X.

Workload (the configuration the headline metric is quoted on): fp16, K = N = 8192,
M in {1, 8, 16}.  One step = one call of each of the six (M, weight layout) combinations:

    fastgemv(W[N,K], x[1,K], y)                 M = 1,  weights [N,K]
    edgemm_m8n128k64x4_bt(A, W_t[N,K], C)       M = 8, 16
    edgemm_m8n128k64x4(A, W[K,N], C)            M = 1, 8, 16, weights [K,N]

through the pybind11 operator surface, on torch's current HIP stream, with all inputs
resident in HBM.  Every call streams a different one of R weight buffers per layout (10
buffers, 1.3 GB in total) so that no weight is served from the 256 MB Infinity Cache.

value = algorithmic bytes of a step / time of a step (GB/s).  Algorithmic bytes of one call:
2*K*N (weights) + 2*M*K (activations) + 2*M*N (result); split-K partials are not counted.

Prints ONE JSON line.  `roofline` describes the kernel that takes the most time in the step,
timed with HIP events on the launch stream; `cpu_baseline` is the reference's CPU path
(torch.matmul with fp32 accumulation on all host cores) on the same step, timed on this host, with
the single-thread C restatement (oracle/fg_oracle.c) nested beside it and labelled as ours;
`configs` carries the benchmark's other configurations (C1-C4) timed the same way.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

K = N = 8192
MS = (1, 8, 16)
R = 5  # weight buffers per layout
HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak

# HBM bytes per launch (`roofline.traffic`) come from bench_traffic.json beside this file: the
# FETCH_SIZE and WRITE_SIZE counters (KiB per dispatch) of two rocprofv3 --pmc runs of this script,
# each scaled by what the same counter reads for kernels of known traffic (--calibrate-traffic: a
# 1 GiB read and a 256 MiB copy).  `bench.py --ingest-pmc DIR` rewrites the file from the CSV output
# of those runs.  Entries are keyed by kernel AND launch plan, so a figure taken under another plan
# is not reported: a call whose key is missing gets null.
TRAFFIC_FILE = ROOT / "bench_traffic.json"


def plan_key(p: dict, M: int) -> str:
    return "%s|M%d|S%d|w%d|f%d|t%d|u%d" % (p["kernel_name"], M, p["splitk"], p["waves"], p["fused"] if p["splitk"] > 1 else 0,
                                           p["tile_n"], p["unroll"])


def load_traffic() -> dict:
    try:
        return json.loads(TRAFFIC_FILE.read_text()).get("entries", {})
    except (OSError, ValueError):
        return {}


def ingest_pmc(directory: Path, capi) -> int:
    """Rewrites bench_traffic.json from DIR/pmc_FETCH_SIZE, DIR/pmc_WRITE_SIZE (this script under
    rocprofv3 --pmc) and DIR/cal_FETCH_SIZE, DIR/cal_WRITE_SIZE (--calibrate-traffic under the same).
    Dispatches are matched to the six calls of the step by kernel family, grid and workgroup size."""
    import csv
    import re

    def rows(sub):
        out = []
        for f in sorted((directory / sub).rglob("*counter_collection.csv")):
            with open(f, newline="") as fh:
                out += list(csv.DictReader(fh))
        return out

    def mean(rs):
        return sum(float(r["Counter_Value"]) for r in rs) / len(rs) if rs else None

    scale = {}
    for counter, known in (("FETCH_SIZE", [("stream_read_kernel", (1 << 30) / 1024.0), ("copyBuffer", (256 << 20) / 1024.0)]),
                           ("WRITE_SIZE", [("copyBuffer", (256 << 20) / 1024.0)])):
        cal = rows("cal_" + counter)
        factors = []
        for frag, true_kib in known:
            got = mean([r for r in cal if frag in r["Kernel_Name"] and r["Counter_Name"] == counter])
            if got:
                factors.append(true_kib / got)
        if not factors:
            print("bench.py: no calibration rows for %s under %s" % (counter, directory), file=sys.stderr)
            return 2
        scale[counter] = sum(factors) / len(factors)
    entries = {}
    for M, layout in ((1, capi.FG_W_NK), (8, capi.FG_W_NK), (16, capi.FG_W_NK), (1, capi.FG_W_KN), (8, capi.FG_W_KN), (16, capi.FG_W_KN)):
        p = capi.plan(M, N, K, layout).as_dict()
        wgs = p["grid_x"] * p["grid_y"] * p["grid_z"]
        vals = {}
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            def match(r):
                # names come demangled (fg::kn_mfma_kernel<2, true, 8>) or mangled (_ZN2fg14kn_mfma_kernelILi2E...)
                if r["Counter_Name"] != counter or not re.search(r"fg(::|\d+)%s_kernel" % p["kernel_name"], r["Kernel_Name"]):
                    return False
                if int(r["Workgroup_Size"]) != p["block"] or int(r["Grid_Size"]) != wgs * p["block"]:
                    return False
                if p["kernel_name"] == "nk_mfma_r":
                    # other calls of the run (M = 8 against 16, the 48-column tiles of another shape) share grid
                    # and block: first template argument = staged activation rows, last = 16-column blocks a tile
                    # (<AROWS, BAND, FULL, NW, CB, ...>; booleans print as words when demangled, as Lb0 / Lb1 when not)
                    m = re.search(r"nk_mfma_r_kernel(<[^>]*>|I\w*?EE)", r["Kernel_Name"])
                    if m is None:
                        return False
                    args = re.findall(r"L[ib](\d+)E", m.group(1)) if m.group(1).startswith("I") else [a.strip() for a in m.group(1)[1:-1].split(",")]
                    return len(args) >= 5 and int(args[0]) == (8 if M <= 8 else 16) and int(args[4]) == p["tile_n"] // 16
                if p["kernel_name"] == "kn_mfma":
                    # <units in flight, waves>: M = 8 and M = 16 may share grid and block
                    m = re.search(r"kn_mfma_kernel(?:<|ILi)(\d+)", r["Kernel_Name"])
                    return m is not None and int(m.group(1)) == p["unroll"]
                return True
            vals[counter] = mean([r for r in rows("pmc_" + counter) if match(r)])
        if vals["FETCH_SIZE"] is None or vals["WRITE_SIZE"] is None:
            print("bench.py: no dispatch matches %s" % plan_key(p, M), file=sys.stderr)
            continue
        entries[plan_key(p, M)] = {
            "fetch_kib": round(vals["FETCH_SIZE"], 1), "write_kib": round(vals["WRITE_SIZE"], 1),
            "bytes": int(round((vals["FETCH_SIZE"] * scale["FETCH_SIZE"] + vals["WRITE_SIZE"] * scale["WRITE_SIZE"]) * 1024)),
            "algorithmic_bytes": algorithmic_bytes(M)}
    TRAFFIC_FILE.write_text(json.dumps({"scale": {k: round(v, 4) for k, v in scale.items()}, "entries": entries}, indent=1) + "\n")
    print(json.dumps({"written": str(TRAFFIC_FILE.name), "entries": len(entries), "scale": scale}))
    return 0


def algorithmic_bytes(M: int) -> int:
    return 2 * K * N + 2 * M * K + 2 * M * N


MODEL_SHAPES = [
    # (label, N, K): projection shapes of common decoder layers, weights [N,K] or [K,N]
    ("7B attn 4096x4096", 4096, 4096), ("7B up 11008x4096", 11008, 4096), ("7B down 4096x11008", 4096, 11008),
    ("13B attn 5120x5120", 5120, 5120), ("13B up 13824x5120", 13824, 5120), ("13B down 5120x13824", 5120, 13824),
    ("8B up 14336x4096", 14336, 4096), ("8B down 4096x14336", 4096, 14336), ("8B qkv 6144x4096", 6144, 4096),
    ("70B attn 8192x8192", 8192, 8192), ("70B up 28672x8192", 28672, 8192), ("70B down 8192x28672", 8192, 28672),
    ("70B kv 1024x8192", 1024, 8192), ("DiT up 12288x3072", 12288, 3072), ("DiT down 3072x12288", 3072, 12288),
]


def run_sweep(torch, sg, capi, dev, steps, warmup, models=False):
    """Per-shape timing of the benchmark configurations: us per call, GB/s on algorithmic bytes,
    fraction of the 8 TB/s peak, and the plan (kernel, split-K, tile) the library chose."""
    import ctypes
    L = capi.lib()

    def time_us(fn):
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps

    # read ceiling for the "fraction of the measured ceiling" column
    probe = [torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256) for _ in range(2)]
    sink = torch.empty(L.fg_stream_read_sink_bytes(), dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    us = time_us(lambda i: L.fg_stream_read(ctypes.c_void_p(probe[i % 2].data_ptr()), 1 << 30,
                                            ctypes.c_void_p(sink.data_ptr()), stream))
    ceiling = (1 << 30) / us / 1e3
    del probe[1]

    # what the same read-only kernel takes for as many bytes as a call moves (whole MiB, rotating over
    # the 1 GiB buffer): launch, ramp-up and tail weigh more the smaller the call
    same_size = {}

    def same_size_read_us(nbytes):
        mib = max(1, min(1024, -(-nbytes // (1 << 20))))
        if mib not in same_size:
            n = mib << 20
            nb = (1 << 30) // n
            base = probe[0].data_ptr()
            fn = lambda i: L.fg_stream_read(ctypes.c_void_p(base + (i % nb) * n), n,
                                            ctypes.c_void_p(sink.data_ptr()), stream)
            same_size[mib] = min(time_us(fn), time_us(fn))
        return same_size[mib]

    def with_same_size(row):
        t = same_size_read_us(row["bytes"])
        row["same_size_read_us"] = round(t, 2)
        row["frac_same_size_read"] = round(t / row["us_per_call"], 4)
        return row

    rows = []

    def fp16_case(name, op, M, Kk, Nn, layout, seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        nbuf = max(2, min(320, -(-(640 << 20) // (2 * Kk * Nn))))  # rotate over > 512 MiB of weights
        shape = (Nn, Kk) if layout == capi.FG_W_NK else (Kk, Nn)
        ws = [(torch.randn(shape, device=dev, generator=g) * 0.02).half() for _ in range(nbuf)]
        a = torch.randn((M, Kk), device=dev, generator=g).half()
        c = torch.zeros((M, Nn), dtype=torch.half, device=dev)
        fn = getattr(sg, op)
        if op.startswith("fastgemv"):
            call = lambda i: fn(ws[i % nbuf], a, c)
        else:
            call = lambda i: fn(a, ws[i % nbuf], c)
        us_call = time_us(call)
        # the vendor GEMM (hipBLASLt through at::matmul_out) on the same buffers, as the reference's
        # scripts print their cuBLAS column
        vend = sg.hgemm_tr if layout == capi.FG_W_NK else sg.hgemm
        c2 = c.view(M, Nn)
        us_vendor = time_us(lambda i: vend(a, ws[i % nbuf], c2))
        by = 2 * Kk * Nn + 2 * M * Kk + 2 * M * Nn
        p = capi.plan(M, Nn, Kk, layout, 0).as_dict()
        rows.append(with_same_size({"config": name, "op": op, "M": M, "K": Kk, "N": Nn,
                     "w_layout": "[N,K]" if layout == capi.FG_W_NK else "[K,N]", "seed": seed,
                     "kernel": p["kernel_name"], "splitk": p["splitk"], "in_launch_reduce": p["fused"],
                     "tile_n": p["tile_n"], "bytes": by, "us_per_call": round(us_call, 2),
                     "GBps": round(by / us_call / 1e3, 1), "TFLOPs": round(2.0 * M * Nn * Kk / us_call / 1e6, 2),
                     "frac_hbm_peak": round(by / us_call / 1e3 / HBM_PEAK_GBPS, 4),
                     "frac_read_ceiling": round(by / us_call / 1e3 / ceiling, 4),
                     "vendor_us_per_call": round(us_vendor, 2)}))

    if models:
        for li, (label, Nn, Kk) in enumerate(MODEL_SHAPES):
            for M in (1, 8, 16):
                fp16_case(label, "edgemm_m8n128k64x4_bt", M, Kk, Nn, capi.FG_W_NK, 3000 + li)
                fp16_case(label, "edgemm_m8n128k64x4", M, Kk, Nn, capi.FG_W_KN, 3000 + li)
        return {"sweep": rows, "read_ceiling_GBps": round(ceiling, 1), "hbm_peak_GBps": HBM_PEAK_GBPS,
                "steps": steps, "warmup": warmup, "data": "synthetic", "dtype": "f16",
                "device": torch.cuda.get_device_name(0)}

    fp16_case("C1 fastgemv", "fastgemv", 1, 4096, 4096, capi.FG_W_NK, 1001)
    fp16_case("C2 edgemm", "edgemm_m8n128k64x4", 8, 4096, 11008, capi.FG_W_KN, 1002)
    fp16_case("C2 edgemm_bt", "edgemm_m8n128k64x4_bt", 8, 4096, 11008, capi.FG_W_NK, 1002)
    fp16_case("C3a flat up-projection", "gemm_m8n128k64x4_bt", 16, 3072, 12288, capi.FG_W_NK, 1003)
    fp16_case("C3b flat down-projection", "gemm_m8n128k64x4_bt", 16, 12288, 3072, capi.FG_W_NK, 1003)
    for ki, kn in enumerate((1024, 4096, 8192, 16384)):
        for mi, M in enumerate((1, 2, 4, 8, 16)):
            seed = 2000 + 16 * ki + mi
            fp16_case("C5 sweep", "edgemm_m8n128k64x4_bt", M, kn, kn, capi.FG_W_NK, seed)
            fp16_case("C5 sweep", "edgemm_m8n128k64x4", M, kn, kn, capi.FG_W_KN, seed)

    # C4: int8 weights, fp16 activations, per-channel scale
    g = torch.Generator(device=dev).manual_seed(1004)
    Kk = Nn = 8192
    wq = [torch.randint(-127, 128, (Nn, Kk), device=dev, generator=g, dtype=torch.int8) for _ in range(10)]
    x = torch.randn((1, Kk), device=dev, generator=g).half()
    scale = (torch.rand(Nn, device=dev, generator=g) * 0.009 + 0.001).half()
    y = torch.empty(Nn, dtype=torch.half, device=dev)
    us_i8 = time_us(lambda i: sg.fastgemv_int8(wq[i % 10], x, y, scale=scale))
    by = Kk * Nn + 2 * Kk + 2 * Nn + 2 * Nn
    us_f16 = next(r["us_per_call"] for r in rows if r["config"] == "C5 sweep" and r["M"] == 1 and r["K"] == 8192
                  and r["w_layout"] == "[N,K]")
    rows.append(with_same_size({"config": "C4 int8 fastgemv", "op": "fastgemv_int8", "M": 1, "K": Kk, "N": Nn, "w_layout": "[N,K] int8",
                 "seed": 1004, "kernel": "wq_m1<int8>", "splitk": 1, "bytes": by, "us_per_call": round(us_i8, 2),
                 "GBps": round(by / us_i8 / 1e3, 1), "frac_hbm_peak": round(by / us_i8 / 1e3 / HBM_PEAK_GBPS, 4),
                 "frac_read_ceiling": round(by / us_i8 / 1e3 / ceiling, 4),
                 "weights_per_ns": round(Kk * Nn / us_i8 / 1e3, 3),
                 "fp16_M1_weights_per_ns": round(Kk * Nn / us_f16 / 1e3, 3),
                 "weight_throughput_vs_fp16": round(us_f16 / us_i8, 3)}))
    # beyond the benchmark's configurations: the int8 GEMV with 4, 8 and 16 activation rows
    for Mb in (4, 8, 16):
        xb = torch.randn((Mb, Kk), device=dev, generator=g).half()
        yb = torch.empty((Mb, Nn), dtype=torch.half, device=dev)
        us_b = time_us(lambda i: sg.fastgemv_int8(wq[i % 10], xb, yb, scale=scale))
        us_fb = next(r["us_per_call"] for r in rows if r["config"] == "C5 sweep" and r["M"] == Mb
                     and r["K"] == 8192 and r["w_layout"] == "[N,K]")
        by = Kk * Nn + 2 * Mb * Kk + 2 * Mb * Nn + 2 * Nn
        rows.append(with_same_size({"config": "extra: int8 batched", "op": "fastgemv_int8", "M": Mb, "K": Kk, "N": Nn,
                     "w_layout": "[N,K] int8", "seed": 1004, "kernel": "w8a16_r", "splitk": 1, "bytes": by,
                     "us_per_call": round(us_b, 2), "GBps": round(by / us_b / 1e3, 1),
                     "frac_hbm_peak": round(by / us_b / 1e3 / HBM_PEAK_GBPS, 4),
                     "frac_read_ceiling": round(by / us_b / 1e3 / ceiling, 4),
                     "weights_per_ns": round(Kk * Nn / us_b / 1e3, 3),
                     "fp16_M1_weights_per_ns": round(Kk * Nn / us_fb / 1e3, 3),
                     "weight_throughput_vs_fp16": round(us_fb / us_b, 3)}))
    # beyond the benchmark's configurations: the same GEMV with 4-bit weights (two per byte)
    del wq
    wq4 = [torch.randint(0, 256, (Nn, Kk // 2), device=dev, generator=g, dtype=torch.uint8) for _ in range(20)]
    us_i4 = time_us(lambda i: sg.fastgemv_int4(wq4[i % 20], x, y, scale=scale, zero_point=8.0))
    by = Kk * Nn // 2 + 2 * Kk + 2 * Nn + 2 * Nn
    rows.append(with_same_size({"config": "extra: int4 fastgemv", "op": "fastgemv_int4", "M": 1, "K": Kk, "N": Nn,
                 "w_layout": "[N,K/2] uint4x2", "seed": 1004, "kernel": "wq_m1<int4>", "splitk": 1, "bytes": by,
                 "us_per_call": round(us_i4, 2), "GBps": round(by / us_i4 / 1e3, 1),
                 "frac_hbm_peak": round(by / us_i4 / 1e3 / HBM_PEAK_GBPS, 4),
                 "frac_read_ceiling": round(by / us_i4 / 1e3 / ceiling, 4),
                 "weights_per_ns": round(Kk * Nn / us_i4 / 1e3, 3),
                 "fp16_M1_weights_per_ns": round(Kk * Nn / us_f16 / 1e3, 3),
                 "weight_throughput_vs_fp16": round(us_f16 / us_i4, 3)}))
    # beyond the benchmark's configurations: [K,N] weights of the metric shape padded to a row pitch
    # of N + 128 elements (a view of a [K, N+128] buffer), as a caller that owns the weights can lay
    # them out once at load time
    g = torch.Generator(device=dev).manual_seed(2040)
    Kp = Np = 8192
    padded = [(torch.randn((Kp, Np + 128), device=dev, generator=g) * 0.02).half() for _ in range(5)]
    views = [w[:, :Np] for w in padded]
    for Mp in (1, 8, 16):
        ap = torch.randn((Mp, Kp), device=dev, generator=g).half()
        cp = torch.zeros((Mp, Np), dtype=torch.half, device=dev)
        us_p = time_us(lambda i: sg.edgemm_m8n128k64x4(ap, views[i % 5], cp))
        us_d = next(r["us_per_call"] for r in rows if r["config"] == "C5 sweep" and r["M"] == Mp
                    and r["K"] == Kp and r["w_layout"] == "[K,N]")
        by = 2 * Kp * Np + 2 * Mp * Kp + 2 * Mp * Np
        pl = capi.plan(Mp, Np, Kp, capi.FG_W_KN, 0).as_dict()
        rows.append(with_same_size({"config": "extra: [K,N] row pitch N+128", "op": "edgemm_m8n128k64x4", "M": Mp, "K": Kp,
                     "N": Np, "w_layout": "[K,N] pitch 8320", "seed": 2040, "kernel": pl["kernel_name"],
                     "splitk": pl["splitk"], "in_launch_reduce": pl["fused"], "tile_n": pl["tile_n"],
                     "bytes": by, "us_per_call": round(us_p, 2), "GBps": round(by / us_p / 1e3, 1),
                     "frac_hbm_peak": round(by / us_p / 1e3 / HBM_PEAK_GBPS, 4),
                     "frac_read_ceiling": round(by / us_p / 1e3 / ceiling, 4),
                     "us_per_call_dense": us_d}))
    del padded, views
    # beyond the benchmark's configurations: the feed-forward pair of C3 (16 x 3072 x 12288, then
    # 16 x 12288 x 3072) with bias and GELU, fused into the two GEMM launches against the same two
    # GEMMs followed by separate elementwise launches
    del wq4
    g = torch.Generator(device=dev).manual_seed(1003)
    Mf, Kf, Nf, nb = 16, 3072, 12288, 5
    w1 = [(torch.randn((Nf, Kf), device=dev, generator=g) * 0.02).half() for _ in range(nb)]
    w2 = [(torch.randn((Kf, Nf), device=dev, generator=g) * 0.02).half() for _ in range(nb)]
    b1 = torch.randn(Nf, device=dev, generator=g).half()
    b2 = torch.randn(Kf, device=dev, generator=g).half()
    af = torch.randn((Mf, Kf), device=dev, generator=g).half()
    hf = torch.empty((Mf, Nf), dtype=torch.half, device=dev)
    cf = torch.empty((Mf, Kf), dtype=torch.half, device=dev)
    us_fused = time_us(lambda i: sg.ffn_bt(af, w1[i % nb], b1, w2[i % nb], b2, hf, cf, "gelu"))

    def unfused(i):
        sg.gemm_m8n128k64x4_bt(af, w1[i % nb], hf)
        h = torch.nn.functional.gelu(hf + b1)
        sg.gemm_m8n128k64x4_bt(h, w2[i % nb], cf)
        cf.add_(b2)

    us_unfused = time_us(unfused)
    by = 2 * (2 * Kf * Nf) + 2 * Mf * Kf * 2 + 2 * Mf * Nf * 2 + 2 * Nf + 2 * Kf
    rows.append(with_same_size({"config": "extra: FFN pair, bias + GELU fused", "op": "ffn_bt", "M": Mf, "K": Kf, "N": Nf,
                 "w_layout": "[N,K] twice", "seed": 1003, "kernel": "nk_mfma_r x2", "splitk": "-", "bytes": by,
                 "us_per_call": round(us_fused, 2), "GBps": round(by / us_fused / 1e3, 1),
                 "frac_hbm_peak": round(by / us_fused / 1e3 / HBM_PEAK_GBPS, 4),
                 "frac_read_ceiling": round(by / us_fused / 1e3 / ceiling, 4),
                 "us_unfused_with_torch_elementwise": round(us_unfused, 2)}))
    return {"sweep": rows, "read_ceiling_GBps": round(ceiling, 1), "hbm_peak_GBps": HBM_PEAK_GBPS,
            "steps": steps, "warmup": warmup, "data": "synthetic", "dtype": "f16",
            "device": torch.cuda.get_device_name(0)}


def run_plan_grid(torch, capi, dev, steps, warmup):
    """The library's plan for each call of the step against explicit alternatives (kernel family x
    split-K x waves x unroll x completion), every one checked against torch.matmul before it is
    timed.  Weights rotate over more than 512 MiB as in the step."""
    import ctypes
    import itertools
    L = capi.lib()
    KN, NK = capi.FG_W_KN, capi.FG_W_NK
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())

    def time_us(fn):
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps

    def candidates(layout, M):
        out = []
        if layout == KN:
            fams = [(capi.FG_KERNEL_KN_MFMA, 16, 0, 0)]
            if M <= 8:
                fams.append((capi.FG_KERNEL_KN_DOT2, M, 0, 0))
            for (kern, mb, tn, band), S, w, U in itertools.product(fams, (2, 4, 8, 16), (4, 8), (1, 2)):
                for fused in ((1, 2, 3) if kern == capi.FG_KERNEL_KN_MFMA else (1, 2)):
                    out.append(dict(kernel=kern, m_block=mb, tile_n=tn, band=band, splitk=S, waves=w, unroll=U,
                                    fused=fused))
        else:
            for tn, band, w, S in itertools.product((16, 32), (128, 256), (4, 8), (1, 2)):
                out.append(dict(kernel=capi.FG_KERNEL_NK_MFMA_R, m_block=16, tile_n=tn, band=band, splitk=S, waves=w,
                                unroll=1, fused=2))
            if M <= 8:
                for tn, U, w, S in itertools.product((4, 8), (1, 2, 4), (4, 8), (1, 2)):
                    out.append(dict(kernel=capi.FG_KERNEL_NK_DOT2, m_block=M, tile_n=tn, band=0, splitk=S, waves=w,
                                    unroll=U, fused=2))
            if M >= 4:
                for tn, U, w, S in itertools.product((8, 16), (1, 2), (4, 8), (1, 2)):
                    out.append(dict(kernel=capi.FG_KERNEL_NK_MFMA4, m_block=(M + 3) // 4 * 4, tile_n=tn, band=0,
                                    splitk=S, waves=w, unroll=U, fused=2))
        return out

    g = torch.Generator(device=dev).manual_seed(2040)
    nbuf = 5
    weights = [(torch.randn((K, N), device=dev, generator=g) * 0.02).half() for _ in range(nbuf)]
    ws = torch.zeros(L.fg_workspace_header_bytes() + (64 << 20), dtype=torch.uint8, device=dev)
    cells = []
    for layout, M in ((NK, 1), (NK, 8), (NK, 16), (KN, 1), (KN, 8), (KN, 16)):
        a = torch.randn((M, K), device=dev, generator=g).half()
        c = torch.empty((M, N), dtype=torch.half, device=dev)
        w0 = weights[0].float()
        ref = a.float() @ (w0 if layout == KN else w0.t())
        lib_plan = capi.plan(M, N, K, layout, 0)

        def timed(plan):
            def fn(i):
                st = L.fg_gemm_f16_planned(vp(a), vp(weights[i % nbuf]), vp(c), M, N, K, layout, 0,
                                           ctypes.byref(plan), vp(ws), ws.numel(), stream)
                if st != 0:
                    raise capi.FastgateError(st, "fg_gemm_f16_planned")
            c.fill_(float("nan"))
            fn(0)
            torch.cuda.synchronize()
            err = float(((c.float() - ref).abs() / (1e-2 + 2e-3 * ref.abs())).max())
            if not err < 1.0:
                raise RuntimeError("plan %r gives wrong results (%.2f)" % (plan.as_dict(), err))
            return min(time_us(fn), time_us(fn))

        rows = []
        for kw in candidates(layout, M):
            q = capi.Plan()
            for k, v in kw.items():
                setattr(q, k, v)
            q.stream_w = lib_plan.stream_w
            try:
                us = timed(q)
            except capi.FastgateError:
                continue          # a combination the kernels do not have
            rows.append(dict(kw, kernel=capi.KERNEL_NAMES[kw["kernel"]], us=round(us, 2)))
        rows.sort(key=lambda r: r["us"])
        us_lib = timed(lib_plan)
        d = lib_plan.as_dict()
        cells.append({"M": M, "N": N, "K": K, "w_layout": "[N,K]" if layout == NK else "[K,N]",
                      "library": {k: d[k] for k in ("kernel_name", "tile_n", "m_block", "band", "splitk", "waves",
                                                    "unroll", "fused")},
                      "library_us": round(us_lib, 2), "alternatives_timed": len(rows), "fastest": rows[:6],
                      "by_split": {str(S): min((r["us"] for r in rows if r["splitk"] == S), default=None)
                                   for S in (1, 2, 4, 8, 16)}})
    return {"plan_grid": cells, "steps": steps, "warmup": warmup, "data": "synthetic", "dtype": "f16",
            "device": torch.cuda.get_device_name(0)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--calibrate-traffic", action="store_true",
                    help="only run kernels of known traffic (1 GiB read probe, 256 MiB device copy) for "
                         "scaling rocprofv3's FETCH_SIZE / WRITE_SIZE counters, then exit")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the headline step, time every benchmark configuration (the fastgemv, "
                         "edgemm, flat-GEMM and int8 shapes and the M x K=N shape sweep on both weight "
                         "layouts) and print one JSON object with the plan and roofline figures per shape")
    ap.add_argument("--sweep-models", action="store_true",
                    help="as --sweep, over the projection shapes of common decoder layers (both layouts, M = 1, 8, 16)")
    ap.add_argument("--plan-grid", action="store_true",
                    help="time the library's plan for each call of the step against explicit alternative plans")
    ap.add_argument("--cpu-repeats", type=int, default=8, help="repetitions of the step on the CPU oracle (0 = skip)")
    ap.add_argument("--ingest-pmc", metavar="DIR", default=None,
                    help="host only: rewrite bench_traffic.json from DIR/{pmc,cal}_{FETCH,WRITE}_SIZE, the CSV output of "
                         "this script and of --calibrate-traffic under rocprofv3 --pmc, then exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU; --gpus %d is not supported "
              "(the path shards by output columns without any collective; each GPU would run this same kernel on its share)" % args.gpus,
              file=sys.stderr)
        return 2

    if args.ingest_pmc:
        from fastgate_amd import capi as capi_host
        return ingest_pmc(Path(args.ingest_pmc), capi_host)

    import numpy as np
    import torch

    import fastgate_amd
    from fastgate_amd import capi

    if not torch.cuda.is_available():
        print("bench.py: no HIP device", file=sys.stderr)
        return 2
    sg = fastgate_amd.speedgate  # ImportError if the extension was not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_traffic:
        import ctypes
        L = capi.lib()
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256)
        sink = torch.empty(L.fg_stream_read_sink_bytes(), dtype=torch.uint8, device=dev)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for _ in range(5):
            L.fg_stream_read(ctypes.c_void_p(src.data_ptr()), 1 << 30, ctypes.c_void_p(sink.data_ptr()), stream)
        a = src[: 256 << 20].view(torch.int32)
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": {"stream_read_kernel": {"read_bytes": 1 << 30, "write_bytes": 0, "launches": 5},
                                          "device_copy_kernel": {"read_bytes": 256 << 20, "write_bytes": 256 << 20,
                                                                 "launches": 5}}}))
        return 0

    if args.plan_grid:
        print(json.dumps(run_plan_grid(torch, capi, dev, args.steps, args.warmup)))
        return 0

    if args.sweep or args.sweep_models:
        print(json.dumps(run_sweep(torch, sg, capi, dev, args.steps, args.warmup, models=args.sweep_models)))
        return 0

    # ---- synthetic inputs, seeded on the CPU so the CPU baseline sees the same bits ----------
    g = torch.Generator().manual_seed(8192)
    acts = {M: torch.randn((M, K), generator=g).half() for M in MS}
    w_nk_host = (torch.randn((N, K), generator=g) * 0.02).half()
    w_nk = [w_nk_host.to(dev)]
    w_kn = [w_nk_host.t().contiguous().to(dev)]
    for r in range(1, R):  # further buffers only have to be distinct memory with the same statistics
        w_nk.append((torch.randn((N, K), device=dev) * 0.02).half())
        w_kn.append((torch.randn((K, N), device=dev) * 0.02).half())
    acts_d = {M: a.to(dev) for M, a in acts.items()}
    outs = {M: torch.empty((M, N), dtype=torch.half, device=dev) for M in MS}
    y1 = torch.empty(N, dtype=torch.half, device=dev)

    calls = []  # (label, M, layout, callable(i))
    calls.append(("fastgemv", 1, capi.FG_W_NK, lambda i: sg.fastgemv(w_nk[i % R], acts_d[1], y1)))
    for M in (8, 16):
        calls.append(("edgemm_m8n128k64x4_bt", M, capi.FG_W_NK,
                      lambda i, M=M: sg.edgemm_m8n128k64x4_bt(acts_d[M], w_nk[i % R], outs[M])))
    for M in MS:
        calls.append(("edgemm_m8n128k64x4", M, capi.FG_W_KN,
                      lambda i, M=M: sg.edgemm_m8n128k64x4(acts_d[M], w_kn[i % R], outs[M])))
    step_bytes = sum(algorithmic_bytes(M) for _, M, _, _ in calls)

    def barrier():
        torch.cuda.synchronize()

    # ---- on-box read ceiling (1 GiB, 16-byte loads) ---------------------------------------------
    L = capi.lib()
    import ctypes
    probe = [torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256) for _ in range(2)]
    sink = torch.empty(L.fg_stream_read_sink_bytes(), dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for i in range(3):
        L.fg_stream_read(ctypes.c_void_p(probe[i % 2].data_ptr()), 1 << 30, ctypes.c_void_p(sink.data_ptr()), stream)
    barrier()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(10):
        L.fg_stream_read(ctypes.c_void_p(probe[i % 2].data_ptr()), 1 << 30, ctypes.c_void_p(sink.data_ptr()), stream)
    e1.record()
    barrier()
    ceiling_gbps = (1 << 30) * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    # device-to-device copy of 1 GiB, counted as read + write bytes (the other usual "copy bandwidth")
    for i in range(2):
        probe[1].copy_(probe[0])
    barrier()
    e0.record()
    for i in range(5):
        probe[1].copy_(probe[0])
    e1.record()
    barrier()
    copy_gbps = 2 * (1 << 30) * 5 / (e0.elapsed_time(e1) * 1e-3) / 1e9

    # the same read-only kernel on as many bytes as one call moves (128 MiB, and 64 MiB for the int8
    # GEMV), rotating over the 1 GiB buffer: what launch, ramp-up and tail leave of the ceiling
    def read_us(n):
        nb = (1 << 30) // n
        fn = lambda i: L.fg_stream_read(ctypes.c_void_p(probe[0].data_ptr() + (i % nb) * n), n,
                                        ctypes.c_void_p(sink.data_ptr()), stream)
        for i in range(10):
            fn(i)
        barrier()
        e0.record()
        for i in range(100):
            fn(i)
        e1.record()
        barrier()
        return e0.elapsed_time(e1) * 1e3 / 100
    read_us_128, read_us_64 = read_us(128 << 20), read_us(64 << 20)
    del probe

    # ---- warm-up, then exactly `steps` timed steps ------------------------------------------------
    it = 0
    for _ in range(args.warmup):
        for _, _, _, fn in calls:
            fn(it)
        it += 1
    ev_a, ev_b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    barrier()
    t0 = time.perf_counter()
    ev_a.record()
    for s in range(args.steps):
        for _, _, _, fn in calls:
            fn(it)
        it += 1
    ev_b.record()
    barrier()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3
    gpu_ms = ev_a.elapsed_time(ev_b)
    ms_per_step = wall_ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- per-call kernel time, outside the timed steps: back-to-back launches of one call between
    # two HIP events on the launch stream (an event between every two calls of the step above would
    # add about 3.5 us of bubble per call and distort `value`).  The launch count does not follow
    # --steps: the gap between the first event and the first kernel (about 10 us) is spread over
    # at least 200 launches after 20 untimed ones, whatever the step count is. -----------------------
    launches = max(args.steps, 200)

    def timed_launches(fn, first=0):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for s_ in range(20):
            fn(first + s_)
        barrier()
        e0.record()
        for s_ in range(launches):
            fn(first + 20 + s_)
        e1.record()
        barrier()
        return e0.elapsed_time(e1) * 1e3 / launches

    per_call = []
    for c, (label, M, layout, fn) in enumerate(calls):
        p = capi.plan(M, N, K, layout).as_dict()
        us = timed_launches(fn, it)
        it += launches + 20
        gbps = algorithmic_bytes(M) / (us * 1e-6) / 1e9
        # the same call on one weight buffer: 128 MiB stays in the 256 MB Infinity Cache
        us_hot = timed_launches(lambda i: fn(0))
        per_call.append({
            "op": label, "M": M, "w_layout": "[N,K]" if layout == capi.FG_W_NK else "[K,N]",
            "kernel": p["kernel_name"], "splitk": p["splitk"], "tile_n": p["tile_n"], "waves": p["waves"],
            "unroll": p["unroll"], "completion": ("second kernel", "counter", "atomic", "flags in one L2", "flags in one L2 (test hook)")[p["fused"]] if p["splitk"] > 1 else "-",
            "plan_key": plan_key(p, M), "launches": 1 + (p["splitk"] > 1 and not p["fused"]),
            "bytes": algorithmic_bytes(M), "us_per_call": round(us, 2), "GBps": round(gbps, 1),
            "us_per_call_single_buffer": round(us_hot, 2),
            "TFLOPs": round(2.0 * M * N * K / (us * 1e-6) / 1e12, 2),
            "frac_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
            "frac_read_ceiling": round(gbps / ceiling_gbps, 4),
            "frac_same_size_read": round(read_us_128 * algorithmic_bytes(M) / (128 << 20) / us, 4)})

    # ---- int8 GEMV (fastgemv_int8, K = N = 8192, per-channel scale) against the fp16 GEMV of the
    # same shape: the two alternate, `launches` back-to-back launches each, five rounds; the ratio of
    # the medians is the int8 path's weight throughput relative to fp16 (target 1.8) ---------------
    gi = torch.Generator(device=dev).manual_seed(1004)
    wq = [torch.randint(-127, 128, (N, K), device=dev, generator=gi, dtype=torch.int8) for _ in range(2 * R)]
    xi = torch.randn((1, K), device=dev, generator=gi).half()
    sc = (torch.rand(N, device=dev, generator=gi) * 0.009 + 0.001).half()
    yi = torch.empty(N, dtype=torch.half, device=dev)

    t_i8, t_f16 = [], []
    for _ in range(5):
        t_f16.append(timed_launches(lambda i: sg.fastgemv(w_nk[i % R], acts_d[1], y1)))
        t_i8.append(timed_launches(lambda i: sg.fastgemv_int8(wq[i % (2 * R)], xi, yi, scale=sc)))
    us_i8, us_f16 = sorted(t_i8)[2], sorted(t_f16)[2]
    i8_bytes = K * N + 2 * K + 2 * N + 2 * N
    int8 = {"op": "fastgemv_int8", "M": 1, "K": K, "N": N, "kernel": "wq_m1<int8>", "bytes": i8_bytes,
            "us_per_call": round(us_i8, 2), "GBps": round(i8_bytes / us_i8 / 1e3, 1),
            "frac_read_ceiling": round(i8_bytes / us_i8 / 1e3 / ceiling_gbps, 4),
            "frac_same_size_read": round(read_us_64 * i8_bytes / (64 << 20) / us_i8, 4),
            "fp16_fastgemv_us_per_call": round(us_f16, 2),
            "weight_throughput_vs_fp16": round(us_f16 / us_i8, 3), "target": 1.8}
    del wq

    # ---- the benchmark's other configurations (C1 fastgemv 4096^2, C2 edgemm 8 x 4096 x 11008 on both
    # layouts, C3 the feed-forward pair at 16 rows, C4 the int8 GEMV), timed like the calls above:
    # rotating over more than 512 MiB of weights, `launches` back-to-back launches after 20 untimed
    # ones, outside the timed steps --------------------------------------------------------------
    def read_us_for(nbytes):
        mib = max(1, -(-nbytes // (1 << 20)))
        n = mib << 20
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256)
        nb = (1 << 30) // n
        t = timed_launches(lambda i: L.fg_stream_read(ctypes.c_void_p(src.data_ptr() + (i % nb) * n), n,
                                                      ctypes.c_void_p(sink.data_ptr()), stream))
        del src
        return t

    def config_row(name, op, M, Kc, Nc, layout, seed):
        gc = torch.Generator(device=dev).manual_seed(seed)
        nbuf = max(2, -(-(640 << 20) // (2 * Kc * Nc)))
        shape = (Nc, Kc) if layout == capi.FG_W_NK else (Kc, Nc)
        wsb = [(torch.randn(shape, device=dev, generator=gc) * 0.02).half() for _ in range(nbuf)]
        a = torch.randn((M, Kc), device=dev, generator=gc).half()
        c = torch.zeros((M, Nc), dtype=torch.half, device=dev)
        f = getattr(sg, op)
        call = (lambda i: f(wsb[i % nbuf], a, c)) if op.startswith("fastgemv") else (lambda i: f(a, wsb[i % nbuf], c))
        us = min(timed_launches(call), timed_launches(call))
        del wsb
        by = 2 * Kc * Nc + 2 * M * Kc + 2 * M * Nc
        pc = capi.plan(M, Nc, Kc, layout).as_dict()
        t_read = read_us_for(by)
        return {"name": name, "op": op, "M": M, "K": Kc, "N": Nc,
                "w_layout": "[N,K]" if layout == capi.FG_W_NK else "[K,N]", "seed": seed, "bytes": by,
                "us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                "frac_hbm_peak": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                "frac_read_ceiling": round(by / us / 1e3 / ceiling_gbps, 4),
                "same_size_read_us": round(t_read, 2), "frac_same_size_read": round(t_read / us, 4),
                "plan_key": plan_key(pc, M)}

    configs = [
        config_row("C1 fastgemv", "fastgemv", 1, 4096, 4096, capi.FG_W_NK, 1001),
        config_row("C2 edgemm", "edgemm_m8n128k64x4", 8, 4096, 11008, capi.FG_W_KN, 1002),
        config_row("C2 edgemm_bt", "edgemm_m8n128k64x4_bt", 8, 4096, 11008, capi.FG_W_NK, 1002),
        config_row("C3a flat up-projection", "gemm_m8n128k64x4_bt", 16, 3072, 12288, capi.FG_W_NK, 1003),
        config_row("C3b flat down-projection", "gemm_m8n128k64x4_bt", 16, 12288, 3072, capi.FG_W_NK, 1003),
        {"name": "C4 int8 fastgemv", "op": "fastgemv_int8", "M": 1, "K": K, "N": N, "w_layout": "[N,K] int8",
         "seed": 1004, "bytes": i8_bytes, "us": int8["us_per_call"], "GBps": int8["GBps"],
         "frac_hbm_peak": round(int8["GBps"] / HBM_PEAK_GBPS, 4), "frac_read_ceiling": int8["frac_read_ceiling"],
         "same_size_read_us": round(read_us_64, 2), "frac_same_size_read": int8["frac_same_size_read"],
         "plan_key": "wq_m1<int8>|M1"},
    ]

    # The roofline entry describes the single-launch call that takes the longest: its time between
    # the events is one kernel's launch-to-launch time, which the rocprofv3 kernel trace must match.
    single = [e for e in per_call if e["launches"] == 1] or per_call
    dom = max(single, key=lambda e: e["us_per_call"])
    roofline = {
        "bound": "hbm", "achieved": dom["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": round(dom["GBps"] / HBM_PEAK_GBPS, 4),
        "traffic": (load_traffic().get(dom["plan_key"]) or {}).get("bytes"),
        "kernel": "%s (%s M=%d %s)" % (dom["kernel"], dom["op"], dom["M"], dom["w_layout"]),
        "launches_in_call": dom["launches"], "us": dom["us_per_call"],
        "algorithmic_bytes": dom["bytes"], "measured_read_ceiling_GBps": round(ceiling_gbps, 1),
        "frac_of_read_ceiling": dom["frac_read_ceiling"],
        "same_size_read_us": {"128MiB": round(read_us_128, 2), "64MiB": round(read_us_64, 2)},
        "frac_of_same_size_read": dom["frac_same_size_read"],
    }

    # ---- CPU baseline: the oracle on the same step -------------------------------------------------
    cpu = None
    if args.cpu_repeats > 0:
        import oracle

        w_nk_np = w_nk_host.numpy()
        w_kn_np = np.ascontiguousarray(w_nk_np.T)
        oracle.gemm_f16(acts[1].numpy()[:, :256], w_nk_np[:128, :256], oracle.W_NK)  # loads the library
        c0 = time.perf_counter()
        for _ in range(args.cpu_repeats):
            for M in MS:
                oracle.gemm_f16(acts[M].numpy(), w_nk_np, oracle.W_NK)
                oracle.gemm_f16(acts[M].numpy(), w_kn_np, oracle.W_KN)
        cpu_s = (time.perf_counter() - c0) / args.cpu_repeats
        torch.set_num_threads(os.cpu_count() or 1)
        a32 = {M: acts[M].float() for M in MS}
        w32 = w_nk_host.float()
        w32t = w32.t().contiguous()
        for M in MS:
            torch.matmul(a32[M], w32.t()), torch.matmul(a32[M], w32t)
        tt = []
        for _ in range(5):
            q0 = time.perf_counter()
            for M in MS:
                torch.matmul(a32[M], w32.t())
                torch.matmul(a32[M], w32t)
            tt.append(time.perf_counter() - q0)
        tm = sorted(tt)[len(tt) // 2]
        cpu = {
            "value": round(step_bytes / tm / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "reference",
            "sample": "the full step (six calls, K=N=8192, M=1/8/16, both weight layouts) through torch.matmul on fp32 "
                      "copies made outside the timed region -- the reference's own CPU check "
                      "(script/standard-test.py:152) -- median of 5 repetitions, %.3f s per step" % tm,
            "s_per_step": round(tm, 4),
            "own_port_single_thread": {
                "value": round(step_bytes / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "note": "ours, not the reference's: oracle/fg_oracle.c (fp32 C loop, one thread) on the same step, "
                        "%d repetitions, %.1f s per step" % (args.cpu_repeats, cpu_s)},
        }

    out = {
        "metric": "achieved HBM GB/s (% of roofline) and us/call, M=1/8/16, K=N=8192 fp16",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "fp16 K=N=8192, M in {1,8,16}, weights [N,K] (fastgemv, edgemm_m8n128k64x4_bt) and "
                               "[K,N] (edgemm_m8n128k64x4): six calls per step, %d rotating weight buffers per layout" % R,
                   "K": K, "N": N, "M": list(MS), "calls_per_step": len(calls), "seed": 8192,
                   "device": torch.cuda.get_device_name(0)},
        "roofline": roofline, "cpu_baseline": cpu,
        "gpu_ms_per_step": round(gpu_ms / args.steps, 4),
        "frac_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "read_ceiling_GBps": round(ceiling_gbps, 1), "frac_read_ceiling": round(value / ceiling_gbps, 4),
        "copy_ceiling_GBps": round(copy_gbps, 1),
        "per_call": per_call,
        "int8_gemv": int8,
        "configs": configs,
        "launches_per_timing": launches,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
