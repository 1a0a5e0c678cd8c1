"""In-tree build of the native pieces.

  libfastgate.so   HIP kernels + C ABI (include/fastgate.h), hipcc --offload-arch=gfx950
  speedgate*.so    pybind11 / ATen host module that mirrors the reference's operator names
                   and forwards to libfastgate (plain C++, no device code)
  fg_cbench        standalone C++ caller of the C ABI (csrc/fg_cbench.cpp): self-check + timing

`python -m fastgate_amd.build` compiles everything; nothing is installed outside the tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
OBJ = ROOT / "build" / "obj"

LIB_NAME = "libfastgate.so"
EXT_NAME = "speedgate" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so")

HIP_SOURCES = [
    "fg_kernels_nk.hip",
    "fg_kernels_kn.hip",
    "fg_kernels_i8.hip",
    "fg_kernels_misc.hip",
    "fg_capi.hip",
]

# plain C++ units of the library (no HIP): the launch planner
HOST_SOURCES = ["fg_planner.cpp"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-Wall",
    "-Wno-unused-function",
    # packed-fp32 VALU forms are kept out of every device code object
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd: list[str], quiet_pattern: str | None = None) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = proc.stdout or ""
    if quiet_pattern:
        out = "\n".join(l for l in out.splitlines() if quiet_pattern not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), out))
    if out.strip():
        print(out.strip(), file=sys.stderr)


def build_lib(verbose: bool = True) -> Path:
    """Compile the HIP translation units in parallel and link libfastgate.so."""
    OBJ.mkdir(parents=True, exist_ok=True)
    hipcc = _hipcc()
    t0 = time.time()

    def compile_one(src: str) -> str:
        obj = OBJ / (Path(src).stem + ".o")
        _run([hipcc, *HIPCC_FLAGS, "-I", str(ROOT / "include"), "-c", str(CSRC / src), "-o", str(obj)],
             quiet_pattern="is not a recognized feature")
        return str(obj)

    def compile_host(src: str) -> str:
        obj = OBJ / (Path(src).stem + ".o")
        _run(["g++", "-O2", "-fPIC", "-std=c++17", "-Wall", "-I", str(ROOT / "include"), "-c", str(CSRC / src),
              "-o", str(obj)])
        return str(obj)

    with ThreadPoolExecutor(max_workers=min(8, len(HIP_SOURCES) + len(HOST_SOURCES))) as pool:
        host = [pool.submit(compile_host, s) for s in HOST_SOURCES]
        objs = list(pool.map(compile_one, HIP_SOURCES)) + [h.result() for h in host]
    out = PKG / LIB_NAME
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(out), *objs])
    if verbose:
        print("built %s in %.1fs" % (out, time.time() - t0), file=sys.stderr)
    return out


def build_ext(verbose: bool = True) -> Path:
    """Compile the pybind11 host module against the installed torch and link it to
    libfastgate.so (found at run time through $ORIGIN)."""
    import torch
    from torch.utils import cpp_extension as ce

    OBJ.mkdir(parents=True, exist_ok=True)
    t0 = time.time()
    torch_lib = Path(torch.__file__).parent / "lib"
    inc = []
    for p in ce.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", sysconfig.get_paths()["include"], "-isystem", "/opt/rocm/include"]
    abi = int(getattr(torch._C, "_GLIBCXX_USE_CXX11_ABI", True))
    obj = OBJ / "speedgate_pybind.o"
    _run(["g++", "-O2", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-variable",
          "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=speedgate",
          "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
          "-I", str(ROOT / "include"), *inc,
          "-c", str(CSRC / "speedgate_pybind.cpp"), "-o", str(obj)])
    out = PKG / EXT_NAME
    _run(["g++", "-shared", "-o", str(out), str(obj),
          "-L", str(PKG), "-l:" + LIB_NAME,
          "-L", str(torch_lib), "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
          "-ltorch_python",
          "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + str(torch_lib)])
    if verbose:
        print("built %s in %.1fs" % (out, time.time() - t0), file=sys.stderr)
    return out


def build_cbench(verbose: bool = True) -> Path:
    """Compile the standalone C++ caller of the C ABI (no torch, no Python)."""
    t0 = time.time()
    out = PKG / "fg_cbench"
    _run([_hipcc(), "-O2", "-std=c++17", "-Wall", "-I", str(ROOT / "include"),
          str(CSRC / "fg_cbench.cpp"), "-o", str(out), "-L", str(PKG), "-l:" + LIB_NAME,
          "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("built %s in %.1fs" % (out, time.time() - t0), file=sys.stderr)
    return out


def build_all() -> None:
    build_lib()
    build_ext()
    build_cbench()


if __name__ == "__main__":
    what = sys.argv[1:] or ["all"]
    if "lib" in what or "all" in what:
        build_lib()
    if "ext" in what or "all" in what:
        build_ext()
    if "cbench" in what or "all" in what:
        build_cbench()
