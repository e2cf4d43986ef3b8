"""Builds the gfx950 operator library (``libdhellam_hip.so``) with hipcc.

The library is plain HIP behind a C ABI (``include/dhellam_hip.h``): no torch
headers, so a cross-compile needs only ROCm.  Objects go to ``build/`` and the
shared object to ``dhellam_amd/lib/`` (in-tree, so it is found next to the
package without installation).

Run as ``python -m dhellam_amd.build``.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libdhellam_hip.so"
OBJ_DIR = ROOT / "build" / "obj"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -packed-fp32-ops is switched off: the compiler would otherwise form packed
# fp32 VALU instructions from scalar float code.
CXXFLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-pragmas",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path, verbose: bool) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [HIPCC, *CXXFLAGS, "-c", str(src), "-o", str(obj)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; drop that line.
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = False, jobs: int | None = None) -> Path:
    """Compile every ``csrc/*.hip`` for gfx950 and link the shared library."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc",
           *map(str, objs), "-lhipblaslt", "-o", str(tmp)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


EXT_SRC = CSRC / "torchapi.cpp"
EXT_PKG = ROOT / "dhellam"


def torch_extension_path() -> Path:
    import sysconfig
    return EXT_PKG / ("_Clib" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_torch_extension(verbose: bool = False) -> Path:
    """Compiles ``csrc/torchapi.cpp`` into the pybind11 torch extension ``dhellam._Clib`` (the reference builds a
    module of that name from its csrc/torchapi.cpp, setup.py:234-244).  Host code only: the host compiler with
    torch's headers, linked against ``libdhellam_hip.so`` (found at run time relative to the extension)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as E
    if not LIB_PATH.exists():
        raise RuntimeError(f"{LIB_PATH} must be built first")
    rocm = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))
    out = torch_extension_path()
    tmp = out.with_suffix(".so.tmp")
    torch_lib = E.library_paths()[0]
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_Clib", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-I{ROOT / 'include'}", *[f"-isystem{p}" for p in E.include_paths()], f"-isystem{rocm / 'include'}",
           f"-I{sysconfig.get_paths()['include']}", str(EXT_SRC), "-o", str(tmp),
           f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python", "-lamdhip64",
           f"-L{LIB_DIR}", "-ldhellam_hip", "-Wl,-rpath,$ORIGIN/../dhellam_amd/lib", f"-Wl,-rpath,{torch_lib}"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"building dhellam._Clib failed:\n{res.stderr}")
    if res.stderr.strip() and verbose:
        print(res.stderr, file=sys.stderr)
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    path = build(verbose="-v" in sys.argv)
    print(path)
    if "--no-ext" not in sys.argv:
        print(build_torch_extension(verbose="-v" in sys.argv))
