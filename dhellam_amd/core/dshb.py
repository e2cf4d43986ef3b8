"""Head block on one rank: word embedding in front of the layers, final norm + output layer +
cross entropy + masked mean loss behind them (dhellam/core/dshb.py:73-112,145-147).

The reference lets autograd differentiate ``post_process``; here forward and backward are
explicit, every step is one of this package's operators, and nothing of size [tokens, vocab]
is kept between them except the logits, which the backward overwrites with their gradient:

  forward   h -> norm -> logits = ln_out @ W^T -> (row max, exp sum, loss per token) -> masked mean
  backward  d loss per token -> d logits (recomputed softmax, written over the logits)
            -> d ln_out = d logits @ W,  W.main_grad += d logits^T @ ln_out -> norm backward

The reference computes the cross entropy on ``logits.float()`` (dshb.py:105): an fp32 copy of
the 16-bit logits.  The kernels read the 16-bit logits and do their arithmetic in fp32, which
gives the same numbers without the copy, and write the gradient in the type the GEMMs take.

Collectives (sequence-parallel all-gather in the output layer, vocab-parallel all-reduces in
the loss) are outside this build: with a tensor-parallel world above one the result is this
rank's share.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..operators.embedding import word_embedding_bwd, word_embedding_fwd
from ..operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
from ..operators.layernorm_column import dgrad_bwd, gemm_fwd, wgrad_bwd
from ..operators.loss import cross_entropy_bwd, cross_entropy_fwd, mask_scale_loss_bwd, mask_scale_loss_fwd


def pre_process(token_ids: torch.Tensor, word_embedding_weight: torch.Tensor, batch_first: bool = False):
    """token ids [b, s] -> hidden states [s, b, h] (dshb.py:138-147), or [b, s, h] with ``batch_first``.
    Returns (hidden, context)."""
    inputs = {"vocab": word_embedding_weight, "token_ids": token_ids}
    out = word_embedding_fwd(inputs)
    emb = out["word_embeddings"]
    return (emb if batch_first else emb.transpose(0, 1).contiguous()), [inputs, out]


def pre_process_bwd(context, d_hidden: torch.Tensor, batch_first: bool = False) -> None:
    """d hidden (layout as returned by ``pre_process``) -> accumulated into the embedding table's gradient."""
    word_embedding_bwd(context, d_hidden if batch_first else d_hidden.transpose(0, 1).contiguous())


def post_process(hidden_states: torch.Tensor, ln_weight: torch.Tensor, ln_bias: Optional[torch.Tensor],
                 labels: torch.Tensor, loss_mask: torch.Tensor, word_embedding_weight: torch.Tensor, num_mb: int,
                 loss_scale: float = 1.0, eps: float = 1e-5, label_smoothing: float = 0.0, batch_first: bool = False):
    """hidden_states [s, b, h] (or [b, s, h] with ``batch_first``), labels / loss_mask [b, s],
    word_embedding_weight [vocab/tp, h].  Returns (loss, context); loss is a 0-d fp32 tensor
    (dshb.py:98-112)."""
    h = hidden_states.shape[-1]
    ln_out, mu, rsigma, _ = pylayernorm_fwd(hidden_states, ln_weight, ln_bias, eps, 0, False, None)
    logits, _ = gemm_fwd(None, ln_out.view(-1, h), word_embedding_weight, None, "TN", False, 0, True, None)
    # the reference's hidden states are sequence-first and its labels batch-first (dshb.py:105)
    target = labels.contiguous() if batch_first else labels.transpose(0, 1).contiguous()
    ce_in = {"vocab_parallel_logits": logits.view(*hidden_states.shape[:2], -1), "target": target}
    ce_out = cross_entropy_fwd(ce_in, label_smoothing, keep_softmax=False)
    token_loss = ce_out["loss"] if batch_first else ce_out["loss"].transpose(0, 1).contiguous()      # [b, s]
    mm_in = {"loss_mask": loss_mask, "output_tensor": token_loss, "num_microbatch": num_mb, "loss_scale": loss_scale}
    mm_out = mask_scale_loss_fwd(mm_in)
    ctx = {"hidden": hidden_states, "ln_weight": ln_weight, "ln_bias": ln_bias, "mu": mu, "rsigma": rsigma,
           "ln_out": ln_out, "weight": word_embedding_weight, "ce": [ce_in, ce_out], "mm": [mm_in, mm_out],
           "batch_first": batch_first}
    return mm_out["loss"], ctx


def post_process_bwd(ctx: Dict) -> torch.Tensor:
    """Backward of ``post_process`` for d loss = 1.  Returns d hidden_states (same layout as given); the
    gradients of the output-layer weight and of the norm parameters are accumulated into their ``main_grad``."""
    h = ctx["hidden"].shape[-1]
    d_token = mask_scale_loss_bwd(ctx["mm"])                                      # [b, s] fp32
    ce_in, ce_out = ctx["ce"]
    logits = ce_in["vocab_parallel_logits"]
    d_rows = d_token if ctx["batch_first"] else d_token.transpose(0, 1).contiguous()
    d_logits = cross_entropy_bwd(ctx["ce"], d_rows, grad_out=logits)
    d2 = d_logits.view(-1, d_logits.shape[-1])
    w = ctx["weight"]
    d_ln_out, _ = dgrad_bwd(None, d2, w, None, "NN", False, 0, True, None)
    wgrad_bwd(None, d2, ctx["ln_out"].view(-1, h), _main_grad(w), True, "NT", False, 0, True, None)
    lw, lb = ctx["ln_weight"], ctx["ln_bias"]
    gw, gb = _main_grad(lw), _main_grad(lb) if lb is not None else None
    fused = gw.dtype == lw.dtype and (gb is None or gb.dtype == lb.dtype)    # the kernel accumulates in the weight's type
    d_hidden, dgamma, dbeta, _ = pylayernorm_bwd(d_ln_out.view(ctx["hidden"].shape), ctx["hidden"], ctx["mu"], ctx["rsigma"], lw, 0,
                                                 False, None, dgamma_out=gw if fused else None,
                                                 dbeta_out=gb if fused else None)
    if not fused:                                                            # fp32 main_grad of a 16-bit parameter
        gw.add_(dgamma)
        if gb is not None:
            gb.add_(dbeta)
    return d_hidden


def _main_grad(p: torch.Tensor) -> torch.Tensor:
    g = getattr(p, "main_grad", None)
    if g is None:
        g = torch.zeros_like(p)
        p.main_grad = g
    return g
