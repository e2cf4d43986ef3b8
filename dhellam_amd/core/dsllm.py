"""Model shell on one rank: word embedding -> L decoder layers -> head, with the micro-batches of
a step paired the reference's way (dhellam/core/dsllm.py:43-106, dhellam/core/dshb.py:114-237):
the first micro-batch runs forward only, then forward of micro-batch i + 1 runs beside backward
of micro-batch i through the whole model, and the last micro-batch runs backward only.

The reference hides this inside Megatron modules and autograd hooks; here it is one explicit
schedule over this package's operators.  In a paired phase the forward strand (stream 1) walks
the layers upward while the backward strand (stream 2) walks them downward, so slot k pairs
forward of layer k with backward of layer L - 1 - k under the plan's DCBlocks:

    stream 1:  embed(i+1)   F_0 ... F_{L-1}(i+1)   head forward(i+1)
    stream 2:  head bwd(i)  B_{L-1} ... B_0(i)     embed bwd(i)

Everything that writes a ``main_grad`` runs on the backward strand.  One rank only
(tensor_model_parallel_size == 1): the collectives between ranks are outside this build.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from . import dshb
from .dstb import DCoperation, LayerConfig, Plan, exec as exec_blocks, init_DCBlocks
from .layer import make_weights


def _record(obj, stream) -> None:
    """Tell the caching allocator that every tensor reachable from ``obj`` is consumed on ``stream``."""
    if isinstance(obj, torch.Tensor):
        if obj.is_cuda:
            obj.record_stream(stream)
    elif isinstance(obj, dict):
        for v in obj.values():
            _record(v, stream)
    elif isinstance(obj, (list, tuple)):
        for v in obj:
            _record(v, stream)


class DSLLM:
    def __init__(self, cfg: LayerConfig, num_layers: int, vocab_size: int, seed: int = 0, plan=None,
                 stream1: Optional[torch.cuda.Stream] = None, stream2: Optional[torch.cuda.Stream] = None,
                 device="cuda"):
        if cfg.tensor_model_parallel_size != 1:
            raise ValueError("the model shell runs one complete rank: tensor_model_parallel_size must be 1")
        self.cfg, self.num_layers = cfg, num_layers
        self.layers: List[Dict[str, torch.Tensor]] = [make_weights(cfg, seed + 1 + l, device) for l in range(num_layers)]
        g = torch.Generator(device="cpu").manual_seed(seed)
        dt = cfg.params_dtype
        self.word_embeddings = (torch.randn(vocab_size, cfg.hidden_size, generator=g) * 0.02).to(dt).to(device)
        self.final_ln_weight = torch.ones(cfg.hidden_size, dtype=dt, device=device)
        for t in (self.word_embeddings, self.final_ln_weight):
            t.main_grad = torch.zeros_like(t)
        self.stream1 = stream1 or torch.cuda.Stream()
        self.stream2 = stream2 or torch.cuda.Stream()
        self.plan: Plan = init_DCBlocks(plan, self.stream1, self.stream2)

    # ---- parameters ---------------------------------------------------------------------------
    def named_parameters(self):
        yield "word_embeddings", self.word_embeddings
        yield "final_ln_weight", self.final_ln_weight
        for l, w in enumerate(self.layers):
            for k, t in w.items():
                if hasattr(t, "main_grad"):
                    yield f"layers.{l}.{k}", t

    def zero_grads(self) -> None:
        for _, t in self.named_parameters():
            t.main_grad.zero_()

    # ---- pieces of a micro-batch --------------------------------------------------------------
    def _exec(self, blocks, fwd_w, bwd_w, x, dy, act_prev, act_new, s1, s2):
        return exec_blocks(self.cfg, DCoperation, fwd_w, bwd_w, x, dy, blocks, s1, s2, act_prev, act_new,
                           movable=self.plan.movable)

    def _embed(self, mb, stream):
        with torch.cuda.stream(stream):
            hidden, ctx = dshb.pre_process(mb["token_ids"], self.word_embeddings, batch_first=True)
        return hidden, ctx

    def _head_fwd(self, mb, hidden, n_mb, loss_scale, stream):
        with torch.cuda.stream(stream):
            loss, ctx = dshb.post_process(hidden, self.final_ln_weight, None, mb["labels"], mb["loss_mask"],
                                          self.word_embeddings, n_mb, loss_scale, self.cfg.layernorm_epsilon,
                                          batch_first=True)
            ctx["_ready"] = torch.cuda.Event()
            ctx["_ready"].record(stream)
        return loss, ctx

    def _head_bwd(self, ctx, stream):
        stream.wait_event(ctx["_ready"])
        _record(ctx, stream)
        with torch.cuda.stream(stream):
            return dshb.post_process_bwd(ctx)

    def _embed_bwd(self, ctx, dx, stream):
        with torch.cuda.stream(stream):
            dshb.pre_process_bwd(ctx, dx, batch_first=True)

    # ---- schedules ----------------------------------------------------------------------------
    def step(self, batches: List[dict], double_strand: bool = True, loss_scale: float = 1.0) -> List[torch.Tensor]:
        """Forward and backward of every micro-batch ({"token_ids", "labels", "loss_mask"}, each [b, s]);
        gradients accumulate into the parameters' ``main_grad``.  Returns the micro-batch losses
        (each already divided by the number of micro-batches and multiplied by ``loss_scale``)."""
        n, L = len(batches), self.num_layers
        s1 = self.stream1
        s2 = self.stream2 if double_strand else self.stream1
        cur = torch.cuda.current_stream()
        s1.wait_stream(cur)
        s2.wait_stream(cur)
        losses: List[torch.Tensor] = [None] * n
        fwd_only, bwd_only, paired = self.plan.fwd_only, self.plan.bwd_only, self.plan.dcblocks

        def forward_alone(i):
            hidden, ectx = self._embed(batches[i], s1)
            acts = [dict() for _ in range(L)]
            for k in range(L):
                hidden, _ = self._exec(fwd_only, self.layers[k], None, hidden, None, None, acts[k], s1, s1)
            losses[i], hctx = self._head_fwd(batches[i], hidden, n, loss_scale, s1)
            return {"embed": ectx, "acts": acts, "head": hctx}

        def backward_alone(state):
            dy = self._head_bwd(state["head"], s2)
            for k in reversed(range(L)):
                _, dy = self._exec(bwd_only, None, self.layers[k], None, dy, state["acts"][k], None, s2, s2)
            self._embed_bwd(state["embed"], dy, s2)

        if not double_strand:
            for i in range(n):
                backward_alone(forward_alone(i))
        else:
            state = forward_alone(0)
            for i in range(1, n):
                hidden, ectx = self._embed(batches[i], s1)
                dy = self._head_bwd(state["head"], s2)
                acts = [dict() for _ in range(L)]
                for k in range(L):
                    kb = L - 1 - k
                    hidden, dy = self._exec(paired, self.layers[k], self.layers[kb], hidden, dy, state["acts"][kb],
                                            acts[k], s1, s2)
                losses[i], hctx = self._head_fwd(batches[i], hidden, n, loss_scale, s1)
                self._embed_bwd(state["embed"], dy, s2)
                state = {"embed": ectx, "acts": acts, "head": hctx}
            backward_alone(state)
        cur.wait_stream(s1)
        cur.wait_stream(s2)
        return losses
