"""bench.py's HBM traffic table: the tracked file has an entry for every plan the library makes
for the calls of the step today (a stale table would print null on the GPU box), and the
ingest of rocprofv3 counter files reproduces a hand-computed figure.  Host only."""
import csv
import importlib.util
import json
import sys
from pathlib import Path

import pytest

from fastgate_amd import capi

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    sys.modules["bench_under_test"] = mod
    spec.loader.exec_module(mod)
    return mod


CALLS = ((1, capi.FG_W_NK), (8, capi.FG_W_NK), (16, capi.FG_W_NK), (1, capi.FG_W_KN), (8, capi.FG_W_KN), (16, capi.FG_W_KN))


def test_tracked_table_covers_the_plans_of_today(bench):
    entries = bench.load_traffic()
    for M, layout in CALLS:
        p = capi.plan(M, bench.N, bench.K, layout).as_dict()
        key = bench.plan_key(p, M)
        assert key in entries, "bench_traffic.json has no entry for %s: re-run the --pmc profile and --ingest-pmc" % key
        e = entries[key]
        assert e["algorithmic_bytes"] == bench.algorithmic_bytes(M)
        # weights read once, little else: within 10 % above the algorithmic bytes, never below
        assert 1.0 <= e["bytes"] / e["algorithmic_bytes"] < 1.10, (key, e)


def _write(path, rows):
    path.parent.mkdir(parents=True, exist_ok=True)
    with open(path, "w", newline="") as fh:
        w = csv.DictWriter(fh, fieldnames=["Kernel_Name", "Counter_Name", "Counter_Value", "Workgroup_Size", "Grid_Size"])
        w.writeheader()
        w.writerows(rows)


def test_ingest_scales_by_the_calibration_kernels(bench, tmp_path, monkeypatch):
    out = tmp_path / "traffic.json"
    monkeypatch.setattr(bench, "TRAFFIC_FILE", out)
    # calibration: FETCH_SIZE reads half of the true bytes, WRITE_SIZE all of them
    _write(tmp_path / "cal_FETCH_SIZE" / "c_counter_collection.csv", [
        dict(Kernel_Name="fg::stream_read_kernel(...)", Counter_Name="FETCH_SIZE", Counter_Value=(1 << 20) / 2, Workgroup_Size=256, Grid_Size=1),
        dict(Kernel_Name="__amd_rocclr_copyBuffer", Counter_Name="FETCH_SIZE", Counter_Value=(256 << 10) / 2, Workgroup_Size=256, Grid_Size=1)])
    _write(tmp_path / "cal_WRITE_SIZE" / "c_counter_collection.csv", [
        dict(Kernel_Name="__amd_rocclr_copyBuffer", Counter_Name="WRITE_SIZE", Counter_Value=256 << 10, Workgroup_Size=256, Grid_Size=1)])
    fetch, write = [], []
    for M, layout in CALLS:
        p = capi.plan(M, bench.N, bench.K, layout).as_dict()
        grid = p["grid_x"] * p["grid_y"] * p["grid_z"] * p["block"]
        # template arguments as the kernels carry them: the row-load kernel <rows, band, full, waves, column
        # blocks, ...>, the [K,N] MFMA kernel <units in flight, waves>
        targs = {"nk_mfma_r": "ILi%dELi128ELb1ELi8ELi%dELb0EEE" % (8 if M <= 8 else 16, p["tile_n"] // 16),
                 "kn_mfma": "ILi%dELi%dEEE" % (p["unroll"], p["waves"])}.get(p["kernel_name"], "ILi%dELi1EEE" % M)
        name = "_ZN2fg%d%s_kernel%svPKDF16_" % (len(p["kernel_name"]) + 7, p["kernel_name"], targs)
        for value in (1000.0 * M, 1002.0 * M):          # two dispatches: the mean counts
            fetch.append(dict(Kernel_Name=name, Counter_Name="FETCH_SIZE", Counter_Value=value, Workgroup_Size=p["block"], Grid_Size=grid))
        write.append(dict(Kernel_Name=name, Counter_Name="WRITE_SIZE", Counter_Value=10.0 * M, Workgroup_Size=p["block"], Grid_Size=grid))
        # a dispatch of the same family with another grid must not be picked up
        fetch.append(dict(Kernel_Name=name, Counter_Name="FETCH_SIZE", Counter_Value=9e9, Workgroup_Size=p["block"], Grid_Size=grid + p["block"]))
    _write(tmp_path / "pmc_FETCH_SIZE" / "c_counter_collection.csv", fetch)
    _write(tmp_path / "pmc_WRITE_SIZE" / "c_counter_collection.csv", write)
    assert bench.ingest_pmc(tmp_path, capi) == 0
    got = json.loads(out.read_text())
    assert got["scale"] == {"FETCH_SIZE": 2.0, "WRITE_SIZE": 1.0}
    keys = set()
    for M, layout in CALLS:
        p = capi.plan(M, bench.N, bench.K, layout).as_dict()
        key = bench.plan_key(p, M)
        keys.add(key)
        if p["kernel_name"] == "nk_mfma_r" and M == 8:
            # M = 8 and M = 16 share grid and block; the template arguments tell them apart
            assert got["entries"][key]["fetch_kib"] == 8008.0
        want = int(round((1001.0 * M * 2.0 + 10.0 * M) * 1024))
        assert got["entries"][key]["bytes"] == want, key
    assert set(got["entries"]) == keys


def test_missing_calibration_is_an_error(bench, tmp_path, monkeypatch):
    monkeypatch.setattr(bench, "TRAFFIC_FILE", tmp_path / "traffic.json")
    assert bench.ingest_pmc(tmp_path, capi) == 2
    assert not (tmp_path / "traffic.json").exists()
