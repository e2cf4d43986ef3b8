"""Model shell on one rank: word embedding -> L decoder layers -> head, with the micro-batches of
a step paired the reference's way (dhellam/core/dsllm.py:43-106, dhellam/core/dshb.py:114-237):
the first micro-batch runs forward only, then forward of micro-batch i + 1 runs beside backward
of micro-batch i through the whole model, and the last micro-batch runs backward only.

Two forms of the same schedule live here.  ``DSLLM`` is the reference's shell: a ``torch.nn.Module`` of
head block + folded ``DSTB`` modules driven by ``model(x1, x2)`` followed by ``.backward()``
on the placeholder it returns (autograd functions and a backward pre-hook move the micro-batches,
``Stack``s hold their activations), without Megatron.  ``DSLLMStep`` is the same thing written as
one explicit schedule over this package's operators.  In a paired phase the forward strand (stream 1) walks
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
from .._Clib import keep_transposed, refresh_transposed
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


class DSLLMStep:
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
        if cfg.resident_weight_transposes:
            keep_transposed(self.word_embeddings)
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
    def step(self, batches: List[dict], double_strand: bool = True, loss_scale: float = 1.0,
             refresh_transposes: bool = True) -> List[torch.Tensor]:
        """Forward and backward of every micro-batch ({"token_ids", "labels", "loss_mask"}, each [b, s]);
        gradients accumulate into the parameters' ``main_grad``.  Returns the micro-batch losses
        (each already divided by the number of micro-batches and multiplied by ``loss_scale``).  The resident
        transposes of the weights are rebuilt first (the weights may have been updated by any means since the last
        step); ``refresh_transposes=False`` is for several calls between two updates."""
        if refresh_transposes and self.cfg.resident_weight_transposes:
            refresh_transposed(t for _, t in self.named_parameters())
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


# ---- the reference's module shell (dsllm.py:10-115) -----------------------------------------------
class Stack:
    def __init__(self):
        self.items = []

    def __str__(self) -> str:
        return f"dhellam.Stack object({len(self.items)} items)"

    def is_empty(self):
        return len(self.items) == 0

    def push(self, item):
        self.items.append(item)

    def pop(self):
        if not self.is_empty():
            return self.items.pop()
        raise IndexError("pop from empty stack")

    def size(self):
        return len(self.items)


def pre_backward_hook(module, grad_output):
    """dsllm.py:108-115: the autograd traversal of a call that took a new micro-batch forward collects that
    micro-batch's second-half activations on a stack of its own."""
    from ..common.global_variables import GLOBAL_VARIABLES
    x1, x2 = GLOBAL_VARIABLES["inputs"]
    if x2 is not None:
        GLOBAL_VARIABLES['bwd_activations'].append(Stack())
    return grad_output


class DSLLM(torch.nn.Module):
    """``num_layers`` decoder layers (even) folded into ``num_layers / 2`` DSTB modules behind a head block
    (dsllm.py:43-106).  One call + backward moves the new micro-batch forward through ALL layers and the
    previous one backward through all of them::

        out = model(previous_loss_or_None, (token_ids, labels, loss_mask) or None); out.backward()

    x1 (the reference passes the previous micro-batch's loss) only says whether a previous micro-batch
    waits for its backward; x2 is the new micro-batch's data.  ``run_microbatches`` drives a whole step.
    One rank (tensor_model_parallel_size == 1), no pipeline stages, no Megatron."""

    def __init__(self, config: LayerConfig, vocab_size: int, num_layers: int, num_mb: int = 1, loss_scale: float = 1.0,
                 seed: int = 0, plan=None, stream1: Optional[torch.cuda.Stream] = None,
                 stream2: Optional[torch.cuda.Stream] = None, pre_process: bool = True, device="cuda"):
        super().__init__()
        from ..common.global_variables import GLOBAL_VARIABLES
        from .dstb import DSTB
        if config.tensor_model_parallel_size != 1:
            raise ValueError("the model shell runs one complete rank: tensor_model_parallel_size must be 1")
        assert num_layers % 2 == 0, "Only support the llm with even number of layers in each pipeline stage!"
        self.config = config
        self.stream1 = stream1 or torch.cuda.Stream()
        self.stream2 = stream2 or torch.cuda.Stream()
        n = num_layers // 2
        # layer l of the network is first_l for l < n and second_{2n-1-l} otherwise; seeds follow the layer number
        self.pre_process = pre_process
        if pre_process:
            self.dchb = dshb.DSHB(config, vocab_size, self.stream1, self.stream2, num_mb, loss_scale, seed, device)
        mods = []
        for k in range(n):
            m = DSTB(config, self.stream1, self.stream2, plan, seed=0, device=device)
            for tag, layer in (("first", k), ("second", 2 * n - 1 - k)):
                w = make_weights(config, seed + 1 + layer, device)
                wd = m.weight_first if tag == "first" else m.weight_second
                with torch.no_grad():
                    for key, p in wd.items():
                        if isinstance(p, torch.nn.Parameter):
                            p.copy_(w[key])
            mods.append(m)
        self.dctb = torch.nn.Sequential(*mods)
        self.input_tensor = None
        GLOBAL_VARIABLES['loss'] = []
        GLOBAL_VARIABLES['fwd_activations'] = []
        GLOBAL_VARIABLES['bwd_activations'] = []
        self.register_full_backward_pre_hook(pre_backward_hook)

    def set_input_tensor(self, input_tensor) -> None:
        self.input_tensor = input_tensor if isinstance(input_tensor, list) else [input_tensor]

    def layer_weights(self, l: int) -> Dict[str, torch.Tensor]:
        """Weight dict of network layer ``l`` (see the folding rule above)."""
        n = len(self.dctb)
        return self.dctb[l].weight_first if l < n else self.dctb[2 * n - 1 - l].weight_second

    def forward(self, x1, x2):
        from ..common.global_variables import GLOBAL_VARIABLES
        if not self.pre_process:
            x1, x2 = self.input_tensor
        backward_only, forward_only = x2 is None, x1 is None
        assert not (forward_only and backward_only), "it's necessary to execute forward pass or backward pass"
        if not backward_only:
            GLOBAL_VARIABLES['fwd_activations'].append(Stack())
        cur = torch.cuda.current_stream()
        self.stream1.wait_stream(cur)
        self.stream2.wait_stream(cur)
        placeholder = torch.zeros(1, dtype=torch.float32, device="cuda", requires_grad=True)
        GLOBAL_VARIABLES['inputs'] = [x1, x2]
        if self.pre_process:
            placeholder = self.dchb(placeholder)
        return self.dctb(placeholder)


def run_microbatches(model: DSLLM, batches: List[dict], refresh_transposes: bool = True) -> List[torch.Tensor]:
    """A whole step through the module shell: forward of micro-batch 0, then forward(i + 1) beside backward(i),
    then the last backward -- the order the reference's patched no-pipelining schedule produces.  Returns the
    micro-batch losses; gradients are in the parameters' ``main_grad``.  The resident transposes of the model's
    weights are rebuilt first: an optimizer that writes through ``p.data`` leaves nothing a lazy check could see."""
    from ..common.global_variables import GLOBAL_VARIABLES
    if refresh_transposes:
        refresh_transposed(model.parameters())
    GLOBAL_VARIABLES['loss'] = []
    prev = None
    for mb in list(batches) + [None]:
        x2 = None if mb is None else (mb["token_ids"], mb["labels"], mb["loss_mask"])
        out = model(prev, x2)
        out.backward()
        prev = GLOBAL_VARIABLES['inputs'][1]           # the new micro-batch's loss (None after the last call)
    cur = torch.cuda.current_stream()
    cur.wait_stream(model.stream1)
    cur.wait_stream(model.stream2)
    return [d['lm loss'] for d in GLOBAL_VARIABLES['loss']]
