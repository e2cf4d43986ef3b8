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

from .._Clib import keep_transposed
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


class DSHB_(torch.autograd.Function):
    """The head block of the folded model (dshb.py:114-237).  Forward traversal: backward of the PREVIOUS
    micro-batch's loss (its gradient becomes the backward strand's input) and the embedding of the NEW one.
    Autograd traversal: the new micro-batch's loss, and the previous micro-batch's embedding gradient."""

    @staticmethod
    def forward(ctx, placeholder, block):
        from ..common.global_variables import GLOBAL_VARIABLES as G
        ctx.block = block
        bwd_input, fwd_input = G['inputs']
        s_f, s_b = block.stream_fwd, block.stream_bwd
        dgrad = fwd_result = None
        with torch.no_grad():
            if bwd_input is not None:
                (head_ctx,) = G['bwd_activations'][0].pop()
                if G['bwd_activations'][0].is_empty():
                    G['bwd_activations'].pop(0)
                s_b.wait_event(head_ctx["_ready"])
                _record_stream(head_ctx, s_b)
                with torch.cuda.stream(s_b):
                    dgrad = post_process_bwd(head_ctx)
            if fwd_input is not None:
                token_ids, labels, loss_mask = fwd_input
                ctx.labels, ctx.loss_mask = labels, loss_mask
                with torch.cuda.stream(s_f):
                    fwd_result, emb_ctx = pre_process(token_ids, block.word_embeddings, batch_first=True)
                G['fwd_activations'][-1].push([emb_ctx])
        G['inputs'] = [dgrad, fwd_result]
        return placeholder.view_as(placeholder)

    @staticmethod
    def backward(ctx, *grads):
        from ..common.global_variables import GLOBAL_VARIABLES as G
        block = ctx.block
        bwd_input, fwd_input = G['inputs']
        s_f, s_b = block.stream_fwd, block.stream_bwd
        loss = None
        with torch.no_grad():
            if bwd_input is not None:
                (emb_ctx,) = G['fwd_activations'][0].pop()
                if G['fwd_activations'][0].is_empty():
                    G['fwd_activations'].pop(0)
                with torch.cuda.stream(s_b):
                    pre_process_bwd(emb_ctx, bwd_input, batch_first=True)
            if fwd_input is not None:
                with torch.cuda.stream(s_f):
                    loss, head_ctx = post_process(fwd_input, block.ln_weight, block.ln_bias, ctx.labels, ctx.loss_mask,
                                                  block.word_embeddings, block.num_mb, block.loss_scale,
                                                  block.config.layernorm_epsilon, batch_first=True)
                    head_ctx["_ready"] = torch.cuda.Event()
                    head_ctx["_ready"].record(s_f)
                G['bwd_activations'][-1].push([head_ctx])
                G['loss'].append({'lm loss': loss})
        G['inputs'] = [None, loss]
        return grads[0], None


def _record_stream(obj, stream) -> None:
    if isinstance(obj, torch.Tensor):
        if obj.is_cuda:
            obj.record_stream(stream)
    elif isinstance(obj, dict):
        for v in obj.values():
            _record_stream(v, stream)
    elif isinstance(obj, (list, tuple)):
        for v in obj:
            _record_stream(v, stream)


class DSHB(torch.nn.Module):
    """Embedding table (tied to the output layer), final norm and loss (dshb.py:239-275), without Megatron's
    ``LanguageModelEmbedding`` / ``ColumnParallelLinear`` and without learned position embeddings (the layers
    rotate q and k instead).  ``num_mb``: micro-batches per step; ``loss_scale``: the reference's
    ``loss_scale_func`` as a factor."""

    def __init__(self, config, vocab_size: int, stream1=None, stream2=None, num_mb: int = 1, loss_scale: float = 1.0,
                 seed: int = 0, device="cuda"):
        super().__init__()
        self.config, self.stream_fwd, self.stream_bwd = config, stream1, stream2
        self.num_mb, self.loss_scale = num_mb, loss_scale
        g = torch.Generator(device="cpu").manual_seed(seed)
        dt = config.params_dtype
        self.word_embeddings = torch.nn.Parameter((torch.randn(vocab_size, config.hidden_size, generator=g) * 0.02).to(dt).to(device))
        self.ln_weight = torch.nn.Parameter(torch.ones(config.hidden_size, dtype=dt, device=device))
        self.ln_bias = None
        for p in (self.word_embeddings, self.ln_weight):
            p.main_grad = torch.zeros_like(p)
        if getattr(config, "resident_weight_transposes", False):
            keep_transposed(self.word_embeddings)      # the logits product's data gradient in the forward's layout
        self.logits_weight = self.word_embeddings

    def forward(self, placeholder):
        return DSHB_.apply(placeholder, self)
