"""The launch planner (fastgate_amd/csrc/fg_planner.cpp, plain C++) built for the host with
AddressSanitizer and UndefinedBehaviorSanitizer and swept over M = 1..64, every N and K that is a
multiple of 128 up to 8192 (of 512 up to 32768, plus the odd projection sizes), both weight
layouts, library plans and forced splits up to 64, for 256, 304 and 64 compute units: no
undefined behaviour, and every plan launchable (tests/planner_sweep.cpp lists the conditions)."""
import subprocess
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_planner_sweep_under_sanitizers(tmp_path):
    exe = tmp_path / "planner_sweep"
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                    "-I", str(ROOT / "include"), "-I", str(ROOT / "fastgate_amd" / "csrc"),
                    str(ROOT / "tests" / "planner_sweep.cpp"), str(ROOT / "fastgate_amd" / "csrc" / "fg_planner.cpp"),
                    "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True, timeout=600,
                         env={"ASAN_OPTIONS": "detect_leaks=1", "UBSAN_OPTIONS": "print_stacktrace=1"})
    assert int(out.stdout.split()[0]) > 5_000_000, out.stdout
