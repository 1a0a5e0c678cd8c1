"""Host-side checks that need no GPU: the C ABI library loads and exports every symbol the
header declares, the launch planner is self-consistent, the pybind11 surface carries every
reference name with the reference's error behaviour, and the product never reaches the oracle."""
import ctypes
import os
import re
import subprocess
from pathlib import Path

import pytest

from fastgate_amd import capi

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "fastgate.h"

KN, NK = capi.FG_W_KN, capi.FG_W_NK
SWEEP = [(M, n, n) for M in (1, 2, 4, 8, 16) for n in (1024, 4096, 8192, 16384)]
CONFIGS = [(1, 4096, 4096), (8, 11008, 4096), (16, 12288, 3072), (16, 3072, 12288), (1, 8192, 8192)]


def _declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(fg_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = _declared()
    assert names == sorted(capi.EXPORTS)
    L = ctypes.CDLL(str(capi.LIB_PATH))
    for n in names:
        assert getattr(L, n) is not None
    assert capi.lib().fg_version() == 110


def test_python_constants_match_the_header():
    text = HEADER.read_text()
    m = re.search(r"#define\s+FG_STATIC_SCRATCH_BYTES\s+\(([^\n]*)\)\s*$", text, flags=re.M)
    assert m and re.fullmatch(r"[0-9 +<()]+", m.group(1))
    assert eval(m.group(1)) == capi.FG_STATIC_SCRATCH_BYTES       # digits, +, << and brackets only
    assert capi.FG_STATIC_SCRATCH_BYTES == capi.lib().fg_workspace_header_bytes() + (8 << 20)
    for name in ("FG_OK", "FG_ERR_INVALID_ARG", "FG_ERR_ALIGN128", "FG_ERR_WORKSPACE", "FG_ERR_LAUNCH",
                 "FG_ERR_UNSUPPORTED", "FG_ERR_SCRATCH_LIMIT", "FG_W_KN", "FG_W_NK"):
        m = re.search(r"\b%s\s*=\s*(-?\d+)" % name, text) or re.search(r"#define\s+%s\s+(-?\d+)" % name, text)
        assert m and int(m.group(1)) == getattr(capi, name), name


_PLAN_ONLY = r"""
import ctypes, os, sys
def state():
    fds = set()
    for f in os.listdir('/proc/self/fd'):
        try:
            fds.add(os.readlink('/proc/self/fd/' + f))
        except OSError:
            pass
    maps = {l.split()[-1] for l in open('/proc/self/maps') if '/' in l}
    threads = len(os.listdir('/proc/self/task'))
    return fds, maps, threads
L = ctypes.CDLL(sys.argv[1])
class Plan(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in ('kernel', 'splitk', 'fused', 'tile_n', 'm_block', 'waves', 'unroll',
                'stream_w', 'stagger', 'band', 'grid_x', 'grid_y', 'grid_z', 'block')] + [('workspace_bytes', ctypes.c_size_t)]
L.fg_plan.argtypes = [ctypes.c_int] * 5 + [ctypes.c_void_p]
L.fg_workspace_bytes.restype = ctypes.c_size_t
before = state()
p = Plan()
for (M, N, K) in ((1, 4096, 4096), (16, 8192, 8192), (8, 11008, 4096)):
    for layout in (0, 1):
        assert L.fg_plan(M, N, K, layout, 0, ctypes.byref(p)) == 0
        assert L.fg_workspace_bytes(M, N, K, layout, 0) == p.workspace_bytes
assert L.fg_compute_units() == 256
L.fg_set_compute_units(304)
assert L.fg_compute_units() == 304
assert L.fg_plan(16, 8192, 8192, 0, 0, ctypes.byref(p)) == 0
after = state()
new_fds = {f for f in after[0] - before[0] if not f.startswith('/proc/')}
assert not new_fds, new_fds
assert not any('kfd' in f or 'renderD' in f for f in after[0]), after[0]
assert after[1] == before[1], after[1] ^ before[1]
assert after[2] == before[2], (before[2], after[2])
print('plan-only process clean')
"""


def _plan_only_process():
    import sys
    out = subprocess.run([sys.executable, "-c", _PLAN_ONLY, str(capi.LIB_PATH)], capture_output=True, text=True,
                         timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "plan-only process clean" in out.stdout


def test_planning_leaves_the_hip_runtime_untouched():
    """A process that loads the library and only plans and sizes buffers opens no device node,
    maps no further library and starts no thread: fg_plan and fg_workspace_bytes are host code."""
    _plan_only_process()


@pytest.mark.gpu
def test_planning_leaves_the_hip_runtime_untouched_with_a_gpu_present():
    _plan_only_process()


def test_header_is_plain_c():
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", str(HEADER)], check=True)


def test_strerror_covers_every_status():
    texts = {capi.strerror(s) for s in (0, -1, -2, -3, -4, -5, -6)}
    assert len(texts) == 7 and all(texts)
    assert "unknown" in capi.strerror(-99)
    assert "128" in capi.strerror(capi.FG_ERR_ALIGN128)


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("M,N,K", SWEEP + CONFIGS + [(3, 128, 128), (33, 256, 384), (7, 1152, 2176)])
def test_plan_is_consistent(layout, M, N, K):
    p = capi.plan(M, N, K, layout)
    d = p.as_dict()
    assert p.kernel in ((capi.FG_KERNEL_KN_DOT2, capi.FG_KERNEL_KN_MFMA) if layout == KN
                        else (capi.FG_KERNEL_NK_DOT2, capi.FG_KERNEL_NK_MFMA4, capi.FG_KERNEL_NK_MFMA_R)), d
    assert N % p.tile_n == 0 and p.grid_x == N // p.tile_n, d
    assert p.grid_y == -(-M // p.m_block) and p.grid_z == p.splitk >= 1, d
    assert p.block == 64 * p.waves and p.waves in (1, 2, 4, 8), d
    hdr = capi.lib().fg_workspace_header_bytes()
    assert p.workspace_bytes == (hdr + p.splitk * M * N * 4 if p.splitk > 1 else 0), d
    assert capi.workspace_bytes(M, N, K, layout) == p.workspace_bytes
    if p.splitk > 1 and p.fused:
        assert p.grid_x * p.grid_y * 4 <= hdr, d   # one counter per output tile
    # v_dot2 is the default for the smallest batches; the MFMA kernels take over above
    if M <= 2 and N * K < 1 << 27:
        assert p.kernel in (capi.FG_KERNEL_KN_DOT2, capi.FG_KERNEL_NK_DOT2), d
    if p.kernel == capi.FG_KERNEL_NK_MFMA_R:
        assert p.tile_n in (16, 32, 48, 64) and p.m_block == (32 if M > 16 else 16), d
    # a forced split is honoured
    for s in (1, 2, 7):
        q = capi.plan(M, N, K, layout, s)
        assert q.splitk == s and q.workspace_bytes == (hdr + s * M * N * 4 if s > 1 else 0)


def test_plan_fills_the_chip_on_the_metric_shapes():
    for layout in (KN, NK):
        for M in (1, 8, 16):
            p = capi.plan(M, 8192, 8192, layout)
            assert p.grid_x * p.grid_y * p.grid_z >= 256, p.as_dict()


def test_plan_choices_that_were_measured():
    # each line is a choice the planner makes because a sweep on the GPU said so; a change here
    # should come with a new measurement
    def nk(M, N, K):
        return capi.plan(M, N, K, NK)

    def kn(M, N, K):
        return capi.plan(M, N, K, KN)

    R = capi.FG_KERNEL_NK_MFMA_R
    # [N,K]: tile widths
    assert (nk(8, 8192, 8192).kernel, nk(8, 8192, 8192).tile_n) == (R, 32)
    assert nk(8, 8192, 4096).tile_n == 16          # rows 8 KB apart: no one-per-CU 32-column tiles
    assert nk(9, 7168, 4096).tile_n == 16          # ... nor 28-column ones
    assert nk(16, 11008, 4096).tile_n == 43        # three column blocks are unaffected
    assert nk(8, 12288, 11008).tile_n == 16        # rows off 2 KB boundaries: no 48-column tiles
    assert nk(8, 12288, 10240).tile_n == 48
    assert nk(4, 9216, 4096).tile_n == 48 and nk(3, 9216, 8192).tile_n == 48
    assert nk(8, 14336, 4096).tile_n == 64 and nk(16, 16384, 8192).tile_n == 64
    # 64 columns from 25/32 of the CUs on, also instead of ragged tiles two a CU (rows on 2 KB boundaries)
    assert nk(8, 12800, 8192).tile_n == 64 and nk(16, 13056, 8192).tile_n == 64 and nk(16, 12800, 8192).tile_n == 64
    assert nk(16, 13824, 4096).tile_n == 64 and nk(16, 13824, 5120).tile_n == 64 and nk(16, 13824, 11008).tile_n == 27
    # 80 tiles of 32 columns split three ways
    p = nk(16, 2560, 8192)
    assert (p.tile_n, p.splitk, p.band) == (32, 3, 128) and nk(8, 2560, 6144).splitk == 3 and nk(8, 2560, 4096).splitk == 1
    assert nk(8, 14336, 2048).tile_n == 32 and nk(8, 14336, 2048).waves == 8
    assert nk(3, 5120, 8192).tile_n == 20
    p = nk(6, 12288, 4096)
    assert (p.tile_n, p.band) == (16, 128)
    # [N,K]: splits of narrow outputs
    assert nk(16, 1024, 6144).splitk > 1 and nk(4, 1024, 6144).splitk == 1
    p = nk(16, 2048, 8192)
    assert (p.tile_n, p.splitk) == (32, 4)
    assert nk(16, 4096, 8192).splitk == 1 and nk(16, 4096, 11008).splitk == 2
    p = nk(16, 3072, 6144)
    assert (p.tile_n, p.splitk) == (48, 4)
    assert nk(9, 3072, 5120).splitk == 1
    # [N,K]: one and two rows
    p = nk(1, 8192, 8192)
    assert (p.kernel, p.unroll, p.stagger) == (capi.FG_KERNEL_NK_DOT2, 1, 0)
    p = nk(1, 4096, 11008)
    assert (p.unroll, p.stagger) == (2, 1)
    p = nk(2, 8192, 16384)
    assert (p.unroll, p.stagger) == (2, 0)
    assert nk(1, 16384, 16384).kernel == capi.FG_KERNEL_NK_MFMA4
    p = nk(1, 5120, 5120)
    assert (p.kernel, p.unroll, p.waves) == (capi.FG_KERNEL_NK_DOT2, 4, 4)   # two and a half steps of four waves made one
    # [K,N]
    # sixteen column tiles or fewer: deep splits (they complete through atomics), four waves for one
    # or two rows from nine tiles on
    for (M, N, K, S, W) in ((1, 2048, 4096, 24, 4), (1, 2048, 16384, 24, 4), (8, 2048, 8192, 16, 8),
                            (1, 1024, 16384, 24, 8), (16, 1024, 28672, 24, 8), (16, 1024, 8192, 24, 8)):
        p = kn(M, N, K)
        assert (p.splitk, p.waves, p.fused) == (S, W, 2), (M, N, K, p.as_dict())
    # one or two rows: v_dot2 up to 2^28 weights (two rows beyond 2^27 only up to N = 12288)
    assert kn(2, 16384, 8192).kernel == capi.FG_KERNEL_KN_MFMA
    assert kn(2, 14336, 16384).kernel == capi.FG_KERNEL_KN_MFMA
    assert kn(1, 16384, 16384).kernel == capi.FG_KERNEL_KN_MFMA
    # widths between the fitted ones with K = 4096 .. 8192: three or four 4-wave workgroups a CU
    for (M, N, K, S, U) in ((1, 6144, 4096, 16, 2), (2, 6144, 8192, 16, 1), (1, 9216, 8192, 14, 1), (1, 10240, 8192, 12, 2),
                            (1, 11008, 4096, 5, 1), (2, 12288, 4096, 10, 1), (1, 12800, 8192, 10, 2), (1, 18432, 4096, 7, 1),
                            (2, 18432, 8192, 7, 1), (1, 22016, 4096, 4, 2), (2, 22016, 8192, 4, 2)):
        p = kn(M, N, K)
        assert (p.kernel, p.splitk, p.waves, p.unroll, p.fused) == (capi.FG_KERNEL_KN_DOT2, S, 4, U, 2), (M, N, K, p.as_dict())
    assert kn(1, 9216, 4096).splitk == 7 and kn(1, 14336, 4096).splitk == 4 and kn(1, 9216, 11008).splitk != 14
    assert kn(1, 28672, 8192).kernel == capi.FG_KERNEL_KN_DOT2
    assert kn(1, 8192, 8192).kernel == capi.FG_KERNEL_KN_DOT2
    for (M, N, K, S) in ((1, 16384, 8192, 8), (1, 8192, 16384, 16), (2, 12288, 16384, 10)):
        p = kn(M, N, K)
        assert (p.kernel, p.splitk, p.waves) == (capi.FG_KERNEL_KN_DOT2, S, 4), (M, N, K, p.as_dict())
    # completion of the split: atomics for v_dot2, for [N,K] and for few elements; the counter otherwise
    assert kn(1, 8192, 8192).fused == 2 and kn(8, 4096, 4096).fused == 2 and nk(16, 2048, 8192).fused == 2
    assert kn(16, 5120, 4096).fused == 1 and kn(8, 14336, 8192).fused == 1
    # the [K,N] MFMA kernel: atomics only for deep splits or few elements (four waves: from 8 splits on)
    assert kn(8, 4096, 8192).fused == 2 and kn(8, 11008, 2048).fused == 2
    # ... and flags in one XCD's L2 where the partials are large, with two or three 4-wave workgroups a
    # CU: (M, N, K) -> (split, waves, units in flight)
    for (M, N, K, S, W, U) in ((8, 8192, 8192, 8, 4, 1), (16, 8192, 8192, 8, 4, 2), (16, 8192, 16384, 8, 4, 2),
                               (8, 12288, 8192, 8, 4, 1), (16, 12288, 12288, 8, 4, 1), (4, 12288, 4096, 8, 4, 1),
                               (16, 4096, 4096, 8, 4, 1), (16, 4096, 11008, 8, 4, 1), (16, 3072, 4096, 8, 4, 1),
                               (16, 2048, 8192, 16, 4, 1), (16, 2048, 16384, 16, 4, 1), (16, 11008, 4096, 5, 4, 1),
                               (8, 11008, 4096, 5, 4, 1), (8, 16384, 2048, 4, 8, 1), (16, 16384, 16384, 2, 4, 1),
                               # 64 tiles from K = 3072 (nine rows and more: 4096) on, 32 tiles with long K
                               (4, 8192, 8192, 8, 4, 1), (4, 8192, 5504, 8, 4, 1), (8, 8192, 4096, 8, 4, 1),
                               (6, 8192, 3072, 8, 4, 1), (16, 8192, 4096, 8, 4, 1), (16, 8192, 6144, 8, 4, 2),
                               (8, 4096, 11008, 8, 4, 1),
                               # widths between the fitted ones: 48 tiles x 9, 80 x 6, 40 x 6, 96 x 8 for short K
                               (16, 6144, 8192, 9, 4, 1), (8, 6144, 4096, 9, 4, 1), (4, 10240, 8192, 6, 4, 1),
                               (16, 10240, 3072, 6, 4, 1), (16, 5120, 8192, 6, 4, 1), (8, 5120, 11008, 6, 4, 1),
                               (8, 12288, 3072, 8, 4, 1), (8, 9216, 4096, 7, 4, 1), (16, 18432, 4096, 5, 4, 1),
                               (8, 22016, 4096, 4, 4, 1), (16, 12800, 8192, 7, 4, 1), (4, 12800, 2048, 4, 4, 1),
                               (4, 20480, 8192, 6, 4, 2), (16, 24576, 8192, 4, 4, 1), (16, 2560, 4096, 8, 8, 1),
                               (16, 3584, 3072, 8, 4, 1)):
        p = kn(M, N, K)
        assert (p.splitk, p.waves, p.unroll, p.fused) == (S, W, U, 3), (M, N, K, p.as_dict())
    # not where the sweep did not go (48 tiles x 6 splits would fill the CUs unevenly) or measured level
    assert kn(16, 6144, 3072).fused != 3 and kn(16, 14336, 8192).fused != 3 and kn(8, 16384, 8192).fused != 3
    assert kn(4, 5120, 8192).fused != 3 and kn(16, 5120, 6144).fused != 3 and kn(8, 10240, 2048).fused != 3
    assert kn(4, 8192, 2048).fused != 3 and kn(16, 8192, 3072).fused != 3 and kn(4, 4096, 11008).fused != 3
    assert kn(24, 2048, 4096).fused == 0           # more than 16 rows: second kernel
    p = kn(16, 5120, 6144)
    assert (p.splitk, p.waves) == (6, 8)
    p = kn(12, 4096, 2048)
    assert (p.splitk, p.waves, p.fused) == (8, 4, 3)    # 7.65 us against 8.34 for four splits of 8 waves and the counter
    assert kn(16, 2048, 2048).splitk == 8
    # one or two rows: two 4-wave workgroups a CU where that lands on 448..512 workgroups
    for (N, K, S) in ((8192, 14336, 8), (8192, 4096, 8), (16384, 5120, 4), (4096, 11008, 16), (10240, 4096, 6)):
        p = kn(1, N, K)
        assert (p.splitk, p.waves) == (S, 4), (N, K, p.as_dict())
    p = kn(1, 4096, 4096)
    assert (p.splitk, p.waves) == (16, 4)          # two units a wave are enough: 8.03 us against 8.29
    p = kn(1, 4096, 3072)
    assert (p.splitk, p.waves) == (8, 8)           # one and a half are not
    p = kn(2, 12288, 4096)
    assert (p.splitk, p.waves) == (10, 4)          # 19.1 us; two splits of 8 waves 19.7 (four would fill the CUs unevenly)
    # small problems (4 Mi weights or fewer), fitted to per-launch times inside a replayed graph:
    # [K,N] v_dot2 on two rows a workgroup with one unit a wave, the MFMA kernel with flags for nine
    # rows and more beyond 1 Mi weights; [N,K] eight waves, narrow outputs split four ways
    D, F = capi.FG_KERNEL_KN_DOT2, capi.FG_KERNEL_KN_MFMA
    for (M, N, K, kern, mb, S, W, fused) in ((1, 1024, 1024, D, 1, 8, 4, 2), (8, 1024, 1024, D, 2, 8, 4, 2),
                                             (16, 1024, 1024, D, 2, 8, 4, 2), (8, 1024, 2048, D, 2, 16, 4, 2),
                                             (16, 2048, 512, D, 2, 4, 4, 2), (4, 2048, 2048, D, 2, 16, 4, 2),
                                             (16, 2048, 1024, F, 16, 8, 4, 3), (16, 1024, 2048, F, 16, 8, 8, 3),
                                             (16, 2048, 2048, F, 16, 8, 8, 3), (8, 4096, 1024, F, 16, 8, 4, 3),
                                             (16, 1024, 4096, F, 16, 16, 8, 3)):
        p = kn(M, N, K)
        assert (p.kernel, p.m_block, p.splitk, p.waves, p.fused) == (kern, mb, S, W, fused), (M, N, K, p.as_dict())
    for (M, N, K, S, band, fused) in ((8, 1024, 1024, 4, 128, 2), (16, 1024, 2048, 4, 128, 2), (4, 1024, 4096, 4, 256, 2),
                                      (16, 512, 2048, 4, 128, 2), (8, 2048, 1024, 1, 128, 0), (16, 4096, 1024, 1, 128, 0)):
        p = nk(M, N, K)
        assert (p.kernel, p.waves, p.splitk, p.band, p.fused) == (R, 8, S, band, fused), (M, N, K, p.as_dict())
    assert nk(8, 2048, 2048).splitk == 1 and nk(8, 2048, 2048).band == 256


def test_plan_rejects_bad_arguments():
    L = capi.lib()
    p = capi.Plan()
    assert L.fg_plan(8, 200, 256, KN, 0, ctypes.byref(p)) == capi.FG_ERR_ALIGN128
    assert L.fg_plan(8, 256, 200, NK, 0, ctypes.byref(p)) == capi.FG_ERR_ALIGN128
    assert L.fg_plan(0, 256, 256, KN, 0, ctypes.byref(p)) == capi.FG_ERR_INVALID_ARG
    assert L.fg_plan(8, 256, 256, 2, 0, ctypes.byref(p)) == capi.FG_ERR_INVALID_ARG
    assert L.fg_plan(8, 256, 256, KN, -1, ctypes.byref(p)) == capi.FG_ERR_INVALID_ARG
    assert L.fg_plan(8, 256, 256, KN, 0, None) == capi.FG_ERR_INVALID_ARG
    assert L.fg_workspace_bytes(8, 200, 256, KN, 0) == 0
    with pytest.raises(capi.FastgateError, match="128"):
        capi.plan(8, 200, 256, KN)


def test_compute_entry_points_validate_before_touching_the_device():
    # argument errors are reported without a device; nothing here launches a kernel
    L = capi.lib()
    one = ctypes.c_void_p(16)
    assert L.fg_gemm_f16(None, one, one, 8, 256, 256, KN, 0, 0, None, 0, None) == capi.FG_ERR_INVALID_ARG
    assert L.fg_gemm_f16(one, one, one, 8, 256, 100, KN, 0, 0, None, 0, None) == capi.FG_ERR_ALIGN128
    assert L.fg_gemm_f16(one, one, one, 8, 256, 256, KN, 0, 4, None, 0, None) == capi.FG_ERR_WORKSPACE
    assert L.fg_gemv_w8a16(one, one, None, 1.0, 0.0, one, 0, 256, 256, None) == capi.FG_ERR_INVALID_ARG
    assert L.fg_gemv_w8a16(one, one, None, 1.0, 0.0, one, 1, 256, 130, None) == capi.FG_ERR_ALIGN128
    assert L.fg_gemv_i8i8_i32(one, one, None, 1, 256, 256, None) == capi.FG_ERR_INVALID_ARG
    assert L.fg_stream_read(one, 24, one, None) == capi.FG_ERR_INVALID_ARG
    assert L.fg_stream_read_sink_bytes() >= 4
    bad = capi.Plan()
    bad.kernel, bad.tile_n, bad.m_block, bad.waves, bad.unroll, bad.splitk = capi.FG_KERNEL_NK_DOT2, 5, 1, 4, 1, 1
    assert L.fg_gemm_f16_planned(one, one, one, 1, 256, 256, NK, 0, ctypes.byref(bad), None, 0, None) == capi.FG_ERR_UNSUPPORTED
    bad.tile_n, bad.kernel = 8, capi.FG_KERNEL_KN_MFMA
    assert L.fg_gemm_f16_planned(one, one, one, 1, 256, 256, NK, 0, ctypes.byref(bad), None, 0, None) == capi.FG_ERR_UNSUPPORTED


# ---- pybind11 surface ---------------------------------------------------------------------------
REFERENCE_NAMES = {
    # backend/cuda/hk/edgemm.h:4-14
    "edgemm", "edgemm_m8n256k64", "edgemm_m8n128k64", "edgemm_m8n128k128", "edgemv_m1n128k64x4",
    "edgemm_m8n128k64x4", "edgemm_m8n128k64x4_bt", "edgemv_m1n256k64x4", "edgemm_m8n128k64x4_amd",
    "edgemm_m8n256k32x8", "edgemm_m8n128k64x4_tr_amd",
    # backend/cuda/hk/flatgemm.h:4-10
    "flat_gemm_m8n128k64x4_bz1", "flat_gemm_m8n256k32x8_bz1", "flat_gemm_m8n256k64x8",
    "flat_gemm_m8n256k32x16", "flat_gemm_m8n512k32x16", "flat_gemm_m8n64k128x8", "flat_gemm_m8n32k256x8",
    # backend/cuda/hk/edgemm_tr.h:7-11
    "gemm_m8n128k64x4_bt", "gemm_m8n32k128x8_bt", "gemm_m8n32k256x8_bt", "gemm_m8n32k256x8_bt_bz2",
    "gemm_m8n64k128x8_bt_exp",
    # backend/cuda/hk/fastgemv.h:4-7, backend/pybind.cpp:23-26
    "fastgemv", "fastgemv_int8", "fastgemv_tuned", "fastgemv_extend", "hgemm", "fastgemm", "mma",
}


@pytest.fixture(scope="module")
def sg():
    import fastgate_amd

    return fastgate_amd.speedgate


def test_every_reference_name_is_bound(sg):
    missing = sorted(n for n in REFERENCE_NAMES if not hasattr(sg, n))
    assert not missing, missing


def test_operator_table_matches_the_oracle_table(sg):
    import oracle

    for name, (layout, protocol, has_bz) in oracle.GEMM_OPS.items():
        doc = getattr(sg, name).__doc__
        assert (", bz:" in doc) == has_bz, name
        assert ("C +=" in doc) == (protocol == "accumulate"), (name, doc)
        assert ("B_t[N,K]" in doc) == (layout == oracle.W_NK), (name, doc)


def test_alignment_error_is_value_error_and_comes_first(sg):
    import torch

    h = torch.half
    C = torch.zeros((8, 128), dtype=h)
    with pytest.raises(ValueError, match="must be multiple of 128"):
        sg.edgemm_m8n128k64x4(torch.zeros((8, 100), dtype=h), torch.zeros((100, 128), dtype=h), C)
    with pytest.raises(ValueError, match="transposed output row"):
        sg.edgemm_m8n128k64x4_bt(torch.zeros((8, 128), dtype=h), torch.zeros((100, 128), dtype=h), C)
    with pytest.raises(ValueError, match="must be multiple of 128"):
        sg.flat_gemm_m8n256k64x8(torch.zeros((8, 100), dtype=h), torch.zeros((100, 128), dtype=h), C, 8)
    with pytest.raises(ValueError, match="must be multiple of 128"):
        sg.gemm_m8n128k64x4_bt(torch.zeros((8, 128), dtype=h), torch.zeros((64, 128), dtype=h), C)
    with pytest.raises(ValueError, match="must be multiple of 128"):
        sg.fastgemv(torch.zeros((128, 64), dtype=h), torch.zeros((1, 64), dtype=h), torch.zeros(128, dtype=h))


def test_no_cpu_path(sg):
    import torch

    h = torch.half
    A, B, C = torch.zeros((8, 128), dtype=h), torch.zeros((128, 128), dtype=h), torch.zeros((8, 128), dtype=h)
    for name in ("edgemm_m8n128k64x4", "edgemm_m8n128k64x4_bt", "gemm_m8n128k64x4_bt", "flat_gemm_m8n256k32x16"):
        with pytest.raises(RuntimeError, match="HIP device"):
            getattr(sg, name)(A, B, C)
    with pytest.raises(RuntimeError, match="HIP device"):
        sg.fastgemv(B, A[:1], torch.zeros(128, dtype=h))
    with pytest.raises(RuntimeError, match="HIP device"):
        sg.fastgemv_int8(B.to(torch.int8), A[:1], torch.zeros(128, dtype=h))
    with pytest.raises(TypeError):
        sg.flat_gemm_m8n256k64x8(A, B, C)  # bz is a required argument, as in the reference


def test_plan_is_reachable_from_python(sg):
    d = sg.plan(16, 8192, 8192, sg.W_NK)
    assert d["grid"][0] * d["grid"][2] >= 256 and d["block"] in (64, 128, 256, 512)
    with pytest.raises(ValueError):
        sg.plan(16, 100, 8192, sg.W_NK)


def test_product_never_touches_the_oracle():
    pkg = ROOT / "fastgate_amd"
    offenders = []
    for path in list(pkg.rglob("*.py")) + list(pkg.rglob("*.hip")) + list(pkg.rglob("*.h")) + list(pkg.rglob("*.cpp")):
        if re.search(r"\boracle\b", path.read_text()):
            offenders.append(str(path.relative_to(ROOT)))
    assert not offenders, offenders


# ---------------------------------------------------------------------------------------
# harness conventions (script/standard-test.py:89-118): which operands each family receives
# ---------------------------------------------------------------------------------------
def _stub(name, log):
    def f(*args):
        log.append((name, args))
    f.__name__ = name
    return f


def test_harness_dispatch_conventions():
    from fastgate_amd import harness
    log = []
    A, B, C, A_T, B_T, C_T = "A", "B", "C", "A_T", "B_T", "C_T"
    harness.dispatch_func(_stub("fastgemv", log), A, B, C, A_T, B_T, C_T)
    harness.dispatch_func(_stub("edgemm_m8n128k64x4_bt", log), A, B, C, A_T, B_T, C_T)
    harness.dispatch_func(_stub("edgemm_m8n128k64x4", log), A, B, C, A_T, B_T, C_T)
    assert log == [("fastgemv", (B_T, A_T, C_T)), ("edgemm_m8n128k64x4_bt", (A, B_T, C)),
                   ("edgemm_m8n128k64x4", (A, B, C))]

    class T:  # stands in for a tensor: transpose().contiguous() yields the [K,N] weight
        def transpose(self, a, b):
            return self
        def contiguous(self):
            return "B"
    log.clear()
    harness.dispatch_func_btrans(_stub("fastgemv_tuned", log), A, B_T, C, 2)
    harness.dispatch_func_btrans(_stub("gemm_m8n32k256x8_bt", log), A, B_T, C, 2)
    harness.dispatch_func_btrans(_stub("gemm_m8n64k128x8_bt_exp", log), A, B_T, C, 2)
    harness.dispatch_func_btrans(_stub("flat_gemm_m8n256k64x8", log), A, T(), C, 4)
    harness.dispatch_func_btrans(_stub("edgemm_m8n256k32x8", log), A, T(), C, 4)
    assert log == [("fastgemv_tuned", (B_T, A, C)), ("gemm_m8n32k256x8_bt", (A, B_T, C)),
                   ("gemm_m8n64k128x8_bt_exp", (A, B_T, C, 2)), ("flat_gemm_m8n256k64x8", (A, "B", C, 4)),
                   ("edgemm_m8n256k32x8", (A, "B", C))]


def test_harness_tables_match_the_bound_operators(sg):
    from fastgate_amd import harness
    bound = set(n for n in dir(sg) if not n.startswith("_"))
    aliases = {"edgemm_m8n32k128x8_bt", "edgemm_m8n32k256x8_bt", "edgemm_m8n64k128x8_bt_tuning",
               "edgemm_m8n32k256x8_bt_tuning"}
    for name in harness.ALL_TRANSPOSED + harness.B_TRANSPOSED + harness.TAKES_BZ:
        assert name in bound or name in aliases, name
    # every [N,K]-layout GEMM name of the semantics table is routed as "B transposed"
    from oracle import oracle
    for name, (layout, _protocol, has_bz) in oracle.GEMM_OPS.items():
        assert (name in harness.B_TRANSPOSED) == (layout == NK), name
        assert (name in harness.TAKES_BZ) == has_bz, name


def test_eed_backend_reexports_every_operator(sg):
    import eed.backend as backend
    for name in dir(sg):
        if not name.startswith("_"):
            assert getattr(backend, name) is getattr(sg, name), name
    assert backend.edgemm_m8n64k128x8_bt_tuning is sg.gemm_m8n64k128x8_bt_exp
    with pytest.raises(ImportError):
        from eed.backend import hgemm_warp2  # noqa: F401  (no surviving definition in the reference)


def test_row_count_beyond_the_grid_limit_is_rejected():
    import ctypes
    p = capi.Plan()
    # [N,K] weights: 32 rows per block row beyond 16 rows; [K,N]: 16
    assert capi.lib().fg_plan(32 * 65535 + 1, 128, 128, capi.FG_W_NK, 0, ctypes.byref(p)) == capi.FG_ERR_INVALID_ARG
    assert capi.lib().fg_plan(32 * 65535, 128, 128, capi.FG_W_NK, 0, ctypes.byref(p)) == capi.FG_OK
    assert capi.lib().fg_plan(16 * 65535 + 1, 128, 128, capi.FG_W_KN, 0, ctypes.byref(p)) == capi.FG_ERR_INVALID_ARG
    assert capi.lib().fg_plan(16 * 65535, 128, 128, capi.FG_W_KN, 0, ctypes.byref(p)) == capi.FG_OK


def test_bz_does_not_change_the_launch(sg):
    """The reference's callers pass bz = 1 or 2 (script/standard-test.py:176), its hosts note
    'orig BZ=2' / 'orig BZ=8' (hk/flatgemm.cu:26,69): split factors of another GPU.  Every
    bz-taking name must run the plan the library picks by itself, and that plan fills the chip."""
    import oracle

    for name, (layout, _protocol, has_bz) in oracle.GEMM_OPS.items():
        if not has_bz:
            continue
        for M in (1, 8, 16):
            auto = sg.plan_for(name, M, 8192, 8192, 0)
            assert auto == sg.plan(M, 8192, 8192, layout, 0)
            for bz in (1, 2, 8):
                assert sg.plan_for(name, M, 8192, 8192, bz) == auto, (name, M, bz)
            gx, gy, gz = auto["grid"]
            assert gx * gy * gz >= 192, (name, M, auto)
    with pytest.raises(ValueError):
        sg.plan_for("flat_gemm_m8n256k64x8", 8, 8192, 8200, 1)
    with pytest.raises(ValueError):
        sg.plan_for("no_such_operator", 8, 8192, 8192, 1)


def test_completion_protocol_can_be_forced_from_the_environment():
    """FASTGATE_SPLITK_COMPLETION is read once per process, so each value gets its own."""
    import sys
    code = ("from fastgate_amd import capi\n"
            "print(capi.plan(1, 8192, 8192, 0).fused, capi.plan(8, 8192, 8192, 0).fused,"
            " capi.plan(64, 8192, 8192, 0).fused, capi.plan(8, 8192, 8192, 0).splitk)")
    seen = {}
    for value in ("", "two-pass", "counter", "atomic", "nonsense"):
        env = dict(os.environ, FASTGATE_SPLITK_COMPLETION=value)
        if not value:
            env.pop("FASTGATE_SPLITK_COMPLETION")
        out = subprocess.run([sys.executable, "-c", code], env=env, cwd=ROOT, capture_output=True, text=True,
                             check=True).stdout.split()
        seen[value] = [int(x) for x in out]
    assert seen[""] == seen["nonsense"]
    assert seen["two-pass"][:2] == [0, 0] and seen["counter"][:2] == [1, 1] and seen["atomic"][:2] == [2, 2]
    assert len({v[3] for v in seen.values()}) == 1       # the split itself is the planner's
