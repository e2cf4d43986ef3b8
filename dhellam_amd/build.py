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


if __name__ == "__main__":
    path = build(verbose="-v" in sys.argv)
    print(path)
