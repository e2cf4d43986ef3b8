"""One decoder layer on the double-strand runtime: weights, micro-batch data, and the
serial / double-strand micro-batch schedules.

The reference builds its layer inside a Megatron module (``DSTB``, dhellam/core/dstb.py:
1283-1468, two weight sets ``*_first`` / ``*_second``) and pairs micro-batches through the
model shell (``DSLLM``, dhellam/core/dsllm.py:43-106): forward-only for the first
micro-batch, forward(i+1) paired with backward(i) in between, backward-only for the last.
This module reproduces that order for one layer on one GPU without Megatron.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .._Clib import keep_transposed, refresh_transposed
from .dstb import DCoperation, LayerConfig, Plan, exec as exec_blocks, init_DCBlocks


def llama70b_tp8_shard(seq_length: int = 4096, micro_batch_size: int = 1, tp_rank: int = 0) -> LayerConfig:
    """One TP=8 / sequence-parallel rank's share of a Llama-3.1-70B decoder layer: hidden
    8192, 64 q heads / 8 kv heads of dim 128 (8 + 1 per rank), SwiGLU FFN 28672 (3584 per
    rank), RoPE theta 5e5, bf16."""
    return LayerConfig(hidden_size=8192, num_attention_heads=64, num_query_groups=8, ffn_hidden_size=28672,
                       seq_length=seq_length, micro_batch_size=micro_batch_size, tensor_model_parallel_size=8,
                       tp_rank=tp_rank, rope_theta=500000.0, params_dtype=torch.bfloat16)


def small_fp32_layer() -> LayerConfig:
    """The fp32 parity configuration: hidden 1024, 16 heads x 64 (MHA), FFN 2816, batch 2,
    seq 512, RoPE theta 1e4."""
    return LayerConfig(hidden_size=1024, num_attention_heads=16, num_query_groups=16, ffn_hidden_size=2816,
                       seq_length=512, micro_batch_size=2, tensor_model_parallel_size=1, rope_theta=10000.0,
                       params_dtype=torch.float32)


def _randn(shape, gen, device, dtype, std=1.0):
    t = torch.randn(shape, generator=gen, dtype=torch.float32, device=gen.device)
    if std != 1.0:
        t = t * std
    return t.to(dtype).to(device)


def make_weights(cfg: LayerConfig, seed: int = 0, device="cuda", gen_device="cpu") -> Dict[str, torch.Tensor]:
    """Weights N(0, 0.02) drawn in fp32 in the fixed order Wqkv, Wo, Wgu, Wd from one
    generator, then cast; norm weights are ones (the reference's init, dstb.py:1393-1394);
    every weight gets a zero ``main_grad`` of its own dtype (dstb.py:1373-1389 keep weights
    and their gradients in one 16-bit type).  Layouts are [out, in] (dstb.py:1374-1379)."""
    g = torch.Generator(device=gen_device).manual_seed(seed)
    h, dt = cfg.hidden_size, cfg.params_dtype
    w = {
        "column_attn_weight": _randn((cfg.qkv_per_rank, h), g, device, dt, 0.02),
        "linear_attn_weight": _randn((h, cfg.heads_per_rank * cfg.head_dim), g, device, dt, 0.02),
        "column_mlp_weight": _randn((2 * cfg.ffn_per_rank, h), g, device, dt, 0.02),
        "linear_mlp_weight": _randn((h, cfg.ffn_per_rank), g, device, dt, 0.02),
        "ln_attn_weight": torch.ones(h, dtype=dt, device=device),
        "ln_mlp_weight": torch.ones(h, dtype=dt, device=device),
    }
    if cfg.layernorm_bias:
        w["ln_attn_bias"] = torch.zeros(h, dtype=dt, device=device)
        w["ln_mlp_bias"] = torch.zeros(h, dtype=dt, device=device)
    for t in w.values():
        t.main_grad = torch.zeros_like(t)
    if cfg.resident_weight_transposes and device != "cpu":
        for k in ("column_attn_weight", "linear_attn_weight", "column_mlp_weight", "linear_mlp_weight"):
            keep_transposed(w[k])
    s = cfg.seq_length
    cu = torch.arange(0, (cfg.micro_batch_size + 1) * s, s, dtype=torch.int32, device=device)
    w["cu_seqlens_q"] = cu
    w["cu_seqlens_kv"] = cu
    if cfg.context_parallel_size > 1:
        # global positions of the rank's local tokens: zig-zag chunks cp_rank and 2 cp - 1 - cp_rank of every sequence
        c, cp, r = s // 2, cfg.context_parallel_size, cfg.cp_rank
        a = torch.arange(c, dtype=torch.int32)
        w["rope_positions"] = torch.cat((r * c + a, (2 * cp - 1 - r) * c + a)).repeat(cfg.micro_batch_size).to(device)
    return w


def make_microbatch(cfg: LayerConfig, seed: int, device="cuda", gen_device="cpu") -> Dict[str, torch.Tensor]:
    """Activations and upstream gradient N(0,1), drawn in the order x, dy, then (sequence
    parallel only) the four peer tensors that stand for the other ranks' rows: P_attn,
    G_attn, P_mlp, G_mlp, each [tokens, hidden], then (context parallel only) the visiting
    KV chunks of the ring."""
    g = torch.Generator(device=gen_device).manual_seed(1000 + seed)
    b, rows, h, dt = cfg.micro_batch_size, cfg.seq_length // cfg.tensor_model_parallel_size, cfg.hidden_size, cfg.params_dtype
    mb = {"x": _randn((b, rows, h), g, device, dt), "dy": _randn((b, rows, h), g, device, dt)}
    if cfg.tensor_model_parallel_size > 1:
        for key in ("sp_peer_attn", "sp_peer_attn_bwd", "sp_peer_mlp", "sp_peer_mlp_bwd"):
            mb[key] = _randn((cfg.tokens, h), g, device, dt)
    if cfg.context_parallel_size > 1:
        # the KV chunks that visit at ring steps 1 .. cp-1, [2, b, 2, s/2, hk, d] each (as their owners rotated them)
        shape = (2, b, 2, cfg.seq_length // 2, cfg.groups_per_rank, cfg.head_dim)
        mb["cp_kv_chunks"] = [_randn(shape, g, device, dt) for _ in range(cfg.context_parallel_size - 1)]
    return mb


def fresh_activation_dict(mb: Dict[str, torch.Tensor]) -> dict:
    """Activation dict of a micro-batch about to start its forward: only the peer buffers and the visiting KV."""
    return {k: v for k, v in mb.items() if k.startswith("sp_peer") or k == "cp_kv_chunks"}


_PROXY = []


def _shared_proxy():
    if not _PROXY:
        from ..common.comm_proxy import CommProxy
        _PROXY.append(CommProxy(2))
    return _PROXY[0]


class LayerRunner:
    """Runs micro-batches through one layer, serially or double-stranded."""

    def __init__(self, cfg: LayerConfig, weights: Dict[str, torch.Tensor], plan=None,
                 stream1: Optional[torch.cuda.Stream] = None, stream2: Optional[torch.cuda.Stream] = None):
        self.proxy = None
        if cfg.comm_standin_engine == "proxy" and cfg.comm_standin_us > 0:
            # the stand-in collectives go to the resident communication proxy (one per process: its flags are
            # signal memory that stays allocated); slot 0 = forward strand, slot 1 = backward strand
            import dataclasses
            self.proxy = cfg.comm_proxy or _shared_proxy()
            cfg = dataclasses.replace(cfg, comm_proxy=self.proxy)
        self.cfg = cfg
        self.weights = weights
        self.stream1 = stream1 or torch.cuda.Stream()
        self.stream2 = stream2 or torch.cuda.Stream()
        self.plan: Plan = init_DCBlocks(plan, self.stream1, self.stream2, cfg.context_parallel_size)

    def _exec(self, blocks, x, dy, act_prev, act_new, s1, s2):
        return exec_blocks(self.cfg, DCoperation, self.weights if act_new is not None else None,
                           self.weights if act_prev is not None else None, x, dy, blocks, s1, s2, act_prev, act_new,
                           movable=self.plan.movable)

    def refresh_weight_transposes(self):
        """Rebuilds W^T of every projection weight on the current stream.  ``run_serial`` / ``run_double_strand``
        call it at the start of every step: a step is what lies between two optimizer steps, and an optimizer that
        writes through ``p.data`` (or a raw kernel, or a collective) leaves no trace a lazy check could see."""
        if self.cfg.resident_weight_transposes:
            refresh_transposed(self.weights.values())

    def run_serial(self, mbs: List[dict], refresh_transposes: bool = True):
        """F0 B0 F1 B1 ... on ONE stream with the fwd_only / bwd_only plans.  ``refresh_transposes=False`` is for a
        caller that runs several such calls between two weight updates."""
        if refresh_transposes:
            self.refresh_weight_transposes()
        s = self.stream1
        s.wait_stream(torch.cuda.current_stream())
        self._proxy_begin()
        outs, dxs = [], []
        for mb in mbs:
            act = fresh_activation_dict(mb)
            out, _ = self._exec(self.plan.fwd_only, mb["x"], None, None, act, s, s)
            _, dx = self._exec(self.plan.bwd_only, None, mb["dy"], act, None, s, s)
            outs.append(out)
            dxs.append(dx)
        self._proxy_end(s, s)
        torch.cuda.current_stream().wait_stream(s)
        return outs, dxs

    def run_double_strand(self, mbs: List[dict], refresh_transposes: bool = True):
        """F0 . (F1 || B0) . (F2 || B1) ... B_last: forward strand on stream1, backward strand
        on stream2, paired steps following the plan's DCBlocks."""
        if refresh_transposes:
            self.refresh_weight_transposes()
        s1, s2 = self.stream1, self.stream2
        cur = torch.cuda.current_stream()
        s1.wait_stream(cur)
        s2.wait_stream(cur)
        self._proxy_begin()
        n = len(mbs)
        outs, dxs = [None] * n, [None] * n
        act = fresh_activation_dict(mbs[0])
        outs[0], _ = self._exec(self.plan.fwd_only, mbs[0]["x"], None, None, act, s1, s2)
        for i in range(1, n):
            act_new = fresh_activation_dict(mbs[i])
            outs[i], dxs[i - 1] = self._exec(self.plan.dcblocks, mbs[i]["x"], mbs[i - 1]["dy"], act, act_new, s1, s2)
            act = act_new
        _, dxs[n - 1] = self._exec(self.plan.bwd_only, None, mbs[n - 1]["dy"], act, None, s1, s2)
        self._proxy_end(s1, s2)
        cur.wait_stream(s1)
        cur.wait_stream(s2)
        return outs, dxs

    def _proxy_begin(self):
        """Starts the step's communication proxy (stand-in collectives with ``comm_standin_engine='proxy'``)."""
        if self.proxy is not None:
            self.proxy.launch(self.cfg.comm_standin_us)

    def _proxy_end(self, fwd_stream, bwd_stream):
        """Ends it: no request follows what the two strands' streams hold now."""
        if self.proxy is not None:
            self.proxy.stop([fwd_stream, bwd_stream])
            torch.cuda.current_stream().wait_stream(self.proxy.stream)

    def zero_grads(self):
        for t in self.weights.values():
            if hasattr(t, "main_grad"):
                t.main_grad.zero_()

    def grads(self) -> Dict[str, torch.Tensor]:
        return {k: t.main_grad for k, t in self.weights.items() if hasattr(t, "main_grad")}
