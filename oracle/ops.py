"""Oracle for the bandwidth-bound operators (norm, SwiGLU, RoPE, residual add).

Test infrastructure: eager PyTorch on the CPU.  Every function takes tensors of
any float dtype, computes in ``dtype`` (fp64 unless stated) and returns tensors
of that dtype; callers cast for comparison.
"""
from __future__ import annotations

import torch

F64 = torch.float64


class _PipelineRound(torch.autograd.Function):
    """What a 16-bit pipeline does to a tensor it hands from one operator to the next: the value is
    rounded to the storage type on the way forward, and the gradient that comes back through the same
    hand-over (the output of the next operator's backward) is rounded to it too."""

    @staticmethod
    def forward(ctx, t, store):
        ctx.store = store
        return t.to(store).to(t.dtype)

    @staticmethod
    def backward(ctx, g):
        return g.to(ctx.store).to(g.dtype), None


def pipeline_round(store):
    """t -> t stored as ``store`` (forward value and backward gradient both); the identity for ``store`` None."""
    if store is None:
        return lambda t: t
    return lambda t: _PipelineRound.apply(t, store)


# --------------------------------------------------------------------------------------
# RMSNorm / LayerNorm.  API slot: dhellam/operators/layernorm.py:6-45 (fwd), :47-91 (bwd).
# The arithmetic is TransformerEngine's (un-vendored); this is the textbook definition.
# --------------------------------------------------------------------------------------
def norm_fwd(x, gamma, beta=None, eps=1e-5, zero_centered_gamma=False, dtype=F64):
    """Returns (y, mu, rsigma).  beta None selects RMSNorm (mu is None)."""
    x = x.to(dtype)
    g = gamma.to(dtype) + (1.0 if zero_centered_gamma else 0.0)
    if beta is None:
        rs = torch.rsqrt((x * x).mean(-1) + eps)
        return x * rs[..., None] * g, None, rs
    mu = x.mean(-1)
    xc = x - mu[..., None]
    rs = torch.rsqrt((xc * xc).mean(-1) + eps)
    return xc * rs[..., None] * g + beta.to(dtype), mu, rs


def norm_bwd(dy, x, mu, rsigma, gamma, zero_centered_gamma=False, dtype=F64):
    """Returns (dx, dgamma, dbeta).  mu None selects RMSNorm (dbeta is None).

    xhat = (x - mu) * rs, g = dy * gamma:
      dx     = rs * (g - xhat * mean(g * xhat) - mean(g))   [the mean(g) term only for LayerNorm]
      dgamma = sum_rows dy * xhat,  dbeta = sum_rows dy
    """
    dy, x, rs = dy.to(dtype), x.to(dtype), rsigma.to(dtype)
    gm = gamma.to(dtype) + (1.0 if zero_centered_gamma else 0.0)
    xh = (x - (mu.to(dtype)[..., None] if mu is not None else 0.0)) * rs[..., None]
    g = dy * gm
    c1 = (g * xh).mean(-1, keepdim=True)
    dx = g - xh * c1
    if mu is not None:
        dx = dx - g.mean(-1, keepdim=True)
    dx = dx * rs[..., None]
    cols = x.shape[-1]
    dgamma = (dy * xh).reshape(-1, cols).sum(0)
    dbeta = dy.reshape(-1, cols).sum(0) if mu is not None else None
    return dx, dgamma, dbeta


# --------------------------------------------------------------------------------------
# SwiGLU.  dhellam/operators/swiglu.py:13-16 (fwd: gate = first half of the last dim)
# and :21-26 (bwd).
# --------------------------------------------------------------------------------------
def swiglu_fwd(y, dtype=F64):
    y1, y2 = torch.chunk(y.to(dtype), 2, -1)
    return y1 * torch.sigmoid(y1) * y2


def swiglu_bwd(g, y, dtype=F64):
    y1, y2 = torch.chunk(y.to(dtype), 2, -1)
    g = g.to(dtype)
    s = torch.sigmoid(y1)
    return torch.cat((g * s * (1 + y1 * (1 - s)) * y2, g * y1 * s), -1)


# --------------------------------------------------------------------------------------
# Residual add = bias-dropout-add with the dropout mask identically one.
# dhellam/operators/bda.py:3-12 (the reference's 0.9 factor belongs to its p = 0.1 mask).
# --------------------------------------------------------------------------------------
def bda_fwd(x, residual, dtype=F64):
    return x.to(dtype) + residual.to(dtype)


def bda_bwd(dgrad, dtype=F64):
    """Returns (d_residual, d_input): the add passes the gradient to both branches."""
    d = dgrad.to(dtype)
    return d, d.clone()


# Legacy kernels of the binding surface.
def gelu_tanh(x, dtype=F64):
    """csrc/operators/gelu.cu:10-15."""
    x = x.to(dtype)
    return x * (0.5 + 0.5 * torch.tanh(x * (0.79788456 + 0.03567741 * x * x)))


def bias_mask_add(x, bias, residual, mask=None, dtype=F64):
    """csrc/operators/bda.cu:10-16: out = mask * (x + bias) + residual."""
    m = 1.0 if mask is None else mask.to(dtype)
    return m * (x.to(dtype) + bias.to(dtype)) + residual.to(dtype)


# --------------------------------------------------------------------------------------
# RoPE, rotate-half (Megatron-core / HF-Llama convention).  Not in the reference; slot
# dhellam/core/dstb.py:122-126 (fwd) and :376-382 (bwd).
# --------------------------------------------------------------------------------------
def rope_inv_freq(theta: float, d: int) -> torch.Tensor:
    """fp32 table: theta^(-2j/d) evaluated in fp64 (Python floats) and rounded once to fp32."""
    return torch.tensor([float(theta) ** (-2.0 * j / d) for j in range(d // 2)], dtype=F64).to(torch.float32)


def rope(x, positions, theta, backward=False, dtype=F64):
    """x [tokens, heads, d]; positions int [tokens].

    The angle is the fp32 product pos * inv_freq[j] (one IEEE rounding, the same
    on every machine); cos/sin and the rotation are evaluated in ``dtype``.
    """
    d = x.shape[-1]
    inv = rope_inv_freq(theta, d)
    ang = (positions.to(torch.float32)[:, None] * inv[None, :]).to(dtype)  # [T, d/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    if backward:
        s = -s
    x = x.to(dtype)
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), -1)
