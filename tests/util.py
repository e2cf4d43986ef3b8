"""Helpers shared by the parity tests."""
import torch

# Tolerances of the path: relative L2 error of outputs and gradients against the oracle.
TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}


def rel_err(a: torch.Tensor, ref: torch.Tensor) -> float:
    """||a - ref||_2 / ||ref||_2 in fp64 (0 when both are all-zero)."""
    a = a.detach().to("cpu", torch.float64)
    ref = ref.detach().to("cpu", torch.float64)
    assert a.shape == ref.shape, f"shape {tuple(a.shape)} vs {tuple(ref.shape)}"
    den = ref.norm().item()
    num = (a - ref).norm().item()
    if den == 0.0:
        return num
    return num / den


def assert_close(a, ref, dtype, what="", scale=1.0):
    e = rel_err(a, ref)
    tol = TOL[dtype] * scale
    assert e <= tol, f"{what}: rel err {e:.3e} > {tol:.1e}"
    return e


def randn(shape, dtype, seed, std=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)
