"""Build-time checks that need no GPU."""
import shutil

import pytest


@pytest.mark.skipif(shutil.which("hipcc") is None and not __import__("os").path.exists("/opt/rocm/bin/hipcc"),
                    reason="needs hipcc")
def test_grouped_gemm_loads_are_left_alone_until_used():
    """The chip-filling grouped GEMM issues its global loads from assembly and orders their use by hand: the compiled
    code may not touch a loaded register before its LDS write (no copy, no spill), in any of the ten instantiations
    (NT / NN with and without the split last round, TN; bf16 and fp16).  ``check_grouped_gemm_loops`` compiles the
    source to assembly and verifies that; a violation raises."""
    from dhellam_amd.build import check_grouped_gemm_loops
    assert check_grouped_gemm_loops() == 10
