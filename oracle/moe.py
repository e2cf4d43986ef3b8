"""Oracle for MoE routing, token permutation and the grouped expert FFN.

Test infrastructure.  Index work is numpy integer arithmetic (bit-exact
comparisons); floating point is fp64 numpy / torch.  The reference has no MoE;
the semantics are dropless top-k routing as in Mixtral / Megatron-core:
softmax over experts, top-k, gates renormalised over the selected k (equal to a
softmax over the k selected logits), tokens grouped by expert with a STABLE sort
of the flat (token, slot) assignment list.
"""
from __future__ import annotations

import numpy as np
import torch


def route_topk(logits: np.ndarray, k: int):
    """logits fp32 [T, E] -> (idx int32 [T, k], gates fp64 [T, k]).

    Selection is on the logits themselves (softmax is monotone): descending value,
    ties to the LOWER expert id -- a stable argsort of the negated row."""
    order = np.argsort(-logits, axis=1, kind="stable")[:, :k]
    sel = np.take_along_axis(logits, order, axis=1).astype(np.float64)
    ex = np.exp(sel - sel[:, :1])
    return order.astype(np.int32), ex / ex.sum(1, keepdims=True)


def sort_assignments(topk_idx: np.ndarray, num_experts: int):
    """Flat assignment a = token*k + slot.  Returns (tokens_per_expert [E], expert_offsets
    [E+1], sorted_idx [T*k], dest_row [T*k]); sorted_idx is the stable order by expert id,
    dest_row its inverse permutation."""
    flat = topk_idx.reshape(-1).astype(np.int64)
    sorted_idx = np.argsort(flat, kind="stable").astype(np.int32)
    tpe = np.bincount(flat, minlength=num_experts).astype(np.int32)
    offs = np.concatenate(([0], np.cumsum(tpe))).astype(np.int32)
    dest = np.empty_like(sorted_idx)
    dest[sorted_idx] = np.arange(sorted_idx.size, dtype=np.int32)
    return tpe, offs, sorted_idx, dest


def permute(x: torch.Tensor, sorted_idx, offs, e_lo, e_hi, k, row_scale=None, dtype=torch.float64):
    """Rows of local experts [e_lo, e_hi): permuted[r] = scale * x[sorted_idx[first + r] // k]."""
    first, last = int(offs[e_lo]), int(offs[e_hi])
    a = torch.from_numpy(np.asarray(sorted_idx[first:last], dtype=np.int64))
    out = x.to(dtype)[a // k]
    if row_scale is not None:
        out = out * row_scale.to(dtype).reshape(-1)[a][:, None]
    return out


def unpermute(y: torch.Tensor, dest_row, offs, e_lo, e_hi, tokens, k, gates=None, dtype=torch.float64):
    """out[t] = sum_j w(t, j) * y[dest_row[t*k + j] - first] over local assignments; zeros elsewhere."""
    first, last = int(offs[e_lo]), int(offs[e_hi])
    out = torch.zeros((tokens, y.shape[1]), dtype=dtype)
    dest = np.asarray(dest_row).reshape(tokens, k)
    yy = y.to(dtype)
    for j in range(k):
        rr = torch.from_numpy(dest[:, j].astype(np.int64)) - first
        ok = (rr >= 0) & (rr < last - first)
        w = gates.to(dtype)[:, j] if gates is not None else torch.ones(tokens, dtype=dtype)
        out[ok] += yy[rr[ok]] * w[ok][:, None]
    return out


def gate_grad(dout, y, dest_row, offs, e_lo, e_hi, tokens, k, dtype=torch.float64):
    """dgates[t, j] = <dout[t], y[row(t, j)]> for local assignments, else 0."""
    first, last = int(offs[e_lo]), int(offs[e_hi])
    dest = np.asarray(dest_row).reshape(tokens, k)
    g = torch.zeros((tokens, k), dtype=dtype)
    for j in range(k):
        rr = torch.from_numpy(dest[:, j].astype(np.int64)) - first
        ok = (rr >= 0) & (rr < last - first)
        g[ok, j] = (dout.to(dtype)[ok] * y.to(dtype)[rr[ok]]).sum(-1)
    return g


def grouped_ffn(xp, w1, w2, group_offs, dtype=torch.float64, round_to=None):
    """Per-expert SwiGLU FFN on the permuted rows.  w1 [G, 2F, H] (gate | up halves as in
    dhellam/operators/swiglu.py:15), w2 [G, H, F]; group g owns rows
    [group_offs[g]-group_offs[0], group_offs[g+1]-group_offs[0]).
    ``round_to``: dtype the intermediate h and a are rounded to (what a 16-bit pipeline
    stores between its GEMMs; the gradients that come back through h and a are rounded to it as
    well).  Returns (y, h, a)."""
    base = int(group_offs[0])
    R = int(group_offs[-1]) - base
    F = w2.shape[2]
    h = torch.zeros((R, 2 * F), dtype=dtype, device=xp.device)
    a = torch.zeros((R, F), dtype=dtype, device=xp.device)
    y = torch.zeros((R, w2.shape[1]), dtype=dtype, device=xp.device)
    from .ops import pipeline_round
    rnd = pipeline_round(round_to)
    for g in range(w1.shape[0]):
        r0, r1 = int(group_offs[g]) - base, int(group_offs[g + 1]) - base
        hg = rnd(xp[r0:r1].to(dtype) @ w1[g].to(dtype).T)
        ag = rnd(hg[:, :F] * torch.sigmoid(hg[:, :F]) * hg[:, F:])
        h[r0:r1], a[r0:r1] = hg, ag
        y[r0:r1] = ag @ w2[g].to(dtype).T
    return y, h, a
