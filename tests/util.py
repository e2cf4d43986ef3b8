"""Helpers shared by the parity tests."""
import os

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


# Local bounds that go with the global one (a wrong boundary tile or a wrong last row moves the global L2 ratio of
# a 4096-row tensor by 1e-4 and would pass it): the tensor is cut into up to ROW_BLOCKS blocks of consecutive rows,
# and every block must meet  ||a - ref||_2 <= C_BLOCK tol ||ref||_2  (its own norm; the global RMS if the block
# of the reference is much smaller than average) and  max|a - ref| <= C_MAX tol max|ref|  (maximum over the block,
# or over the tensor if larger).  C_BLOCK = 2 allows a block to be twice as far off as the tensor as a whole;
# C_MAX = 2 allows one element an error of 2 tol of the largest value around it (a value rounded to bf16 is off
# by at most 0.2 % of itself), and never less than one unit in the last place of the storage type.  A block holds
# at least MIN_BLOCK elements (the tiny known-answer vectors are one block: a single row of a few values is noise).
ROW_BLOCKS, C_BLOCK, C_MAX, MIN_BLOCK = 64, 2.0, 2.0, 4096
ULP = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}


def local_err(a: torch.Tensor, ref: torch.Tensor):
    """(worst block L2 ratio, worst max-abs ratio, index of the worst block) under the rules above."""
    a = a.detach().to("cpu", torch.float64)
    ref = ref.detach().to("cpu", torch.float64)
    if a.numel() == 0:
        return 0.0, 0.0, -1
    a2 = a.reshape(-1, a.shape[-1]) if a.dim() > 1 else a.reshape(-1, 1)   # rows = everything but the last dim
    r2 = ref.reshape(a2.shape)
    n = a2.shape[0]
    nb = max(1, min(ROW_BLOCKS, n, a2.numel() // MIN_BLOCK))
    edges = [(i * n) // nb for i in range(nb + 1)]
    g_rms = (r2.pow(2).mean().sqrt().item()) or 1.0
    g_max = r2.abs().max().item() or 1.0
    worst_l2, worst_max, where = 0.0, 0.0, -1
    for i in range(nb):
        d = a2[edges[i]:edges[i + 1]] - r2[edges[i]:edges[i + 1]]
        rb = r2[edges[i]:edges[i + 1]]
        den = max(rb.norm().item(), 0.1 * g_rms * (rb.numel() ** 0.5))
        l2 = d.norm().item() / den
        mx = d.abs().max().item() / max(rb.abs().max().item(), 0.1 * g_max)
        if l2 > worst_l2:
            worst_l2, where = l2, i
        worst_max = max(worst_max, mx)
    return worst_l2, worst_max, where


def assert_close(a, ref, dtype, what="", scale=1.0, local=True):
    e = rel_err(a, ref)
    tol = TOL[dtype] * scale
    if scale > 1.0 and os.environ.get("DH_REPORT_SCALED"):       # which widened bounds are really needed
        print(f"[scaled] {what}: rel err {e:.3e}, base tol {TOL[dtype]:.0e}, scale {scale:g}")
    assert e <= tol, f"{what}: rel err {e:.3e} > {tol:.1e}"
    if local:
        l2, mx, where = local_err(a, ref)
        assert l2 <= C_BLOCK * tol, f"{what}: row block {where} of {ROW_BLOCKS}: rel err {l2:.3e} > {C_BLOCK * tol:.1e}"
        mtol = max(C_MAX * tol, ULP[dtype])
        assert mx <= mtol, f"{what}: max |a - ref| is {mx:.3e} of the largest value around it > {mtol:.1e}"
    return e


def randn(shape, dtype, seed, std=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)
