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


def check_grouped_gemm_loops(verbose: bool = False) -> int:
    """The chip-filling grouped GEMM kernel (``grouped_gemm_w4_kernel``) issues its loads from assembly, so the compiler
    does not know that their results arrive later: the kernel is only correct if, between a load and the LDS write
    that consumes it, NO instruction names the loaded registers (a register copy or a spill there would move data
    that has not arrived).  The source arranges that; this check holds the generated code to it.  It compiles
    ``grouped_gemm.hip`` to device assembly and, in the main loop of every instantiation of the kernel (the innermost
    loop with 32 loads), follows each ``buffer_load_dwordx4`` destination to its ``ds_write_b128`` across the loop's
    back edge; it also refuses scratch accesses and register copies inside that loop.  Returns the number of loops
    checked; raises on a violation."""
    import re
    import tempfile
    with tempfile.TemporaryDirectory() as td:
        out = Path(td) / "gg.s"
        cmd = [HIPCC, *[f for f in CXXFLAGS if f != "-fPIC"], "--cuda-device-only", "-S", str(CSRC / "grouped_gemm.hip"), "-o", str(out)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("hipcc -S failed for grouped_gemm.hip:\n" + res.stderr)
        lines = out.read_text().split("\n")

    def regs(tok: str) -> set:
        m = re.match(r"v\[(\d+):(\d+)\]$", tok)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.match(r"v(\d+)$", tok)
        return {int(m.group(1))} if m else set()

    checked = 0
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN2dh22grouped_gemm_w4_kernel\w+:", l)]
    for a in starts:
        b = next(i for i in range(a, len(lines)) if lines[i].startswith(".Lfunc_end"))   # (a kernel may hold several s_endpgm)
        fn = lines[a:b]
        labels = {m.group(1): i for i, l in enumerate(fn) if (m := re.match(r"^(\.LBB\d+_\d+):", l))}
        loops = []
        for i, l in enumerate(fn):
            m = re.match(r"\s+s_cbranch_\w+ (\.LBB\d+_\d+)", l)
            if m and m.group(1) in labels and labels[m.group(1)] < i:
                body = fn[labels[m.group(1)]:i]
                if sum("buffer_load_dwordx4" in x for x in body) == 32:
                    loops.append(body)
        if not loops:
            raise RuntimeError(f"{fn[0].split(':')[0]}: no main loop with 32 loads found (the kernel's structure changed: "
                               "update check_grouped_gemm_loops)")
        body = min(loops, key=len)
        name = fn[0].split(":")[0]
        for l in body:
            if "scratch_" in l or re.match(r"\s+v_mov_b\d+", l) or "v_accvgpr" in l:
                raise RuntimeError(f"{name}: '{l.strip()}' inside the main loop")
        if sum("v_mfma" in x for x in body) != 128:
            raise RuntimeError(f"{name}: {sum('v_mfma' in x for x in body)} MFMAs in the main loop, expected 128")
        # the same rule from the first load of the function up to the loop (the prologue's loads, whose results the
        # loop's first slices write to LDS) and from the loop's end to the wait for every load that follows it
        lo = next(i for i, l in enumerate(fn) if l is body[0])
        first = next(i for i, l in enumerate(fn) if "buffer_load_dwordx4" in l)
        hi = lo + len(body)
        end = next((i for i in range(hi, len(fn)) if "s_waitcnt vmcnt(0)" in fn[i]), None)
        if first >= lo or end is None:
            raise RuntimeError(f"{name}: prologue loads or the wait behind the loop not found")
        pending: dict = {}
        for n, l in enumerate(fn[first:lo] + body + body + fn[hi:end]):   # the loop twice: values live across the back edge
            t = l.replace(",", " ").split()
            if not t or t[0].startswith((";", ".")):
                continue
            if t[0] == "buffer_load_dwordx4":
                for r in regs(t[1]):
                    if r in pending:
                        raise RuntimeError(f"{name}: v{r} is loaded again before the LDS write of its previous load")
                    pending[r] = n
                continue
            if t[0] == "s_waitcnt" and "vmcnt(0)" in l:     # everything has arrived
                pending.clear()
                continue
            touched = set().union(*[regs(x) for x in t[1:]]) & set(pending)
            if touched:
                if t[0] != "ds_write_b128":
                    raise RuntimeError(f"{name}: '{l.strip()}' names a register whose load may still be in flight")
                for r in touched:
                    pending.pop(r)
        checked += 1
        if verbose:
            print(f"checked {name}: {len(body)} lines", flush=True)
    if checked == 0:
        raise RuntimeError("no grouped_gemm_w4_kernel instantiation found in the assembly")
    return checked


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
    print(f"grouped GEMM main loops checked: {check_grouped_gemm_loops(verbose='-v' in sys.argv)}")
    if "--no-ext" not in sys.argv:
        print(build_torch_extension(verbose="-v" in sys.argv))
