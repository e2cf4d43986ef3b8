"""The C-ABI library loads and exports every symbol the header declares (no GPU needed)."""
import ctypes
import os
import re

from dhellam_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dhellam_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dh_[a-z0-9_]+)\s*\(", text)))


def _ensure_lib():
    if not _lib.LIB_PATH.exists():
        from dhellam_amd.build import build
        build()


def test_header_and_ctypes_table_agree():
    assert _declared_symbols() == sorted(_lib.SIGNATURES), "include/dhellam_hip.h and _lib.SIGNATURES list different symbols"


def test_library_exports_every_declared_symbol():
    _ensure_lib()
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in _declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in the header but missing from the library"


def test_argument_counts_match_header():
    text = open(os.path.join(ROOT, "include", "dhellam_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    for name, (_, args) in _lib.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else len([p for p in params.split(",") if p.strip()])
        assert n == len(args), f"{name}: header has {n} parameters, ctypes table has {len(args)}"


def test_version_and_error_string_without_gpu():
    _ensure_lib()
    lib = _lib.load()
    assert lib.dh_version() >= 100
    # argument validation happens on the host, before any HIP call: usable without a GPU
    rc = lib.dh_norm_fwd(None, None, None, None, None, None, 4, 0, 1e-5, 0, 0, None)
    assert rc == -1
    msg = lib.dh_last_error().decode()
    assert "norm.hip" in msg and "norm_fwd" in msg and "bad shape" in msg
    rc = lib.dh_attn_fwd(None, None, None, None, None, None, None, 1, 8, 8, 5, 2, 64, 0, 0, 0, 0, 1.0, 1, 1, None)
    assert rc == -1 and "multiple" in lib.dh_last_error().decode()
    rc = lib.dh_moe_route_topk(None, None, None, 10, 100, 2, None)
    assert rc == -1 and "experts" in lib.dh_last_error().decode()


def test_product_does_not_import_the_oracle():
    """Nothing under dhellam_amd/ may import, read or run the oracle (it is the checker)."""
    for dirpath, _, files in list(os.walk(os.path.join(ROOT, "dhellam_amd"))) + list(os.walk(os.path.join(ROOT, "dhellam"))):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", src, flags=re.M), f"{f} imports the oracle"
