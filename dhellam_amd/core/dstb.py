"""Double-strand transformer block: op adapters, activation bookkeeping, op graph,
plan loader and the two-stream scheduler.

Counterpart of dhellam/core/dstb.py: ``FuncChoice`` (:24-58), ``DCFunc`` (:64-425),
``DCoperation.perform_operation`` (:427-660), ``DCOP`` / ``DCBlock`` (:662-695),
``init_DCBlocks`` (:698-1131) and ``exec`` (:1133-1281).  Kept: the integer op ids
and op-name strings (they are the vocabulary of plan files and profile records), the
activation-dict keys and their save/free points, the plan JSON schema, the built-in
default plans, the rule "an op without successors defines its strand's result", and
wgrad accumulation into ``weight.main_grad``.

Re-designed for one MI355X:

* Table dispatch instead of a chain of ``if operation == N``.
* No device-wide synchronisation per block.  A strand is one HIP stream, so its ops are
  ordered by the stream; the only cross-stream edge -- backward of micro-batch i reading
  what forward of micro-batch i produced -- is an event that travels inside the
  activation dict (``_ready``).  Tensors consumed on a stream other than the one they
  were allocated on are registered with ``record_stream``.
* The sequence-parallel all-gather / reduce-scatter ops keep their names and places in
  the graph but are single-GPU stand-ins: "gather" writes this rank's rows into the
  micro-batch's pre-generated peer buffer and returns it, "scatter" returns this rank's
  row slice.  With tensor_model_parallel_size == 1 they are the identity.
* RoPE ops (``rope``, ``rope_bwd``) are added to the graph; plans that do not name them
  get them inserted next to ``fl_attn`` / ``attn_bwd``.
* Context parallelism (``context_parallel_size`` = cp > 1): the graph holds the ring steps
  ``cp_attn_block_fwd_1 .. _cp`` and ``cp_attn_block_bwd_1 .. _cp+1`` in place of ``fl_attn`` /
  ``attn_bwd`` (the reference builds them for cp = 2 only, dstb.py:711-722,801-817); the KV
  chunks that would arrive over the ring are the micro-batch's pre-generated
  ``cp_kv_chunks``, nothing is exchanged, and ``seq_length`` is the rank's local length.
* GQA: the fused QKV weight is packed per kv-group as [q heads of the group | k | v]
  (for MHA this is the reference's per-head q|k|v interleave, dstb.py:111-122); with one
  group per rank q, k, v are strided views of the projection output (no copies), and
  dq, dk, dv are written straight into the packed gradient (no concat).
* Norm backward fuses the residual-gradient add and the main_grad accumulation that the
  reference issues as three extra launches (dstb.py:387-405).
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass
from enum import Enum
from typing import List, Optional

import torch

from .. import _lib
from .._Clib import pymha_varlen_bwd, pymha_varlen_fwd, _attn_bwd_raw
from ..operators.bda import bda_bwd, bda_fwd
from ..operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
from ..operators.layernorm_column import dgrad_bwd, gemm_fwd, wgrad_bwd
from ..operators.ring_attn import RingGroup, fa_cp_block_bwd, fa_cp_block_fwd
from ..operators.rope import rope_bwd, rope_fwd
from ..operators.swiglu import swiglu, swiglu_back


class FuncChoice(Enum):
    ln_attn = 1
    ln_mlp = 2
    gemm_attn_column = 3
    gemm_attn_linear = 4
    gemm_mlp_column = 5
    gemm_mlp_linear = 6
    attn = 7
    bda_mlp = 8
    bda_attn = 9
    reduce_scatter = 10
    all_gather = 11
    swiglu = 12
    gemm_dgrad_mlp_c = 13
    gemm_wgrad_mlp_c = 14
    gemm_dgrad_mlp_l = 15
    gemm_wgrad_mlp_l = 16
    gemm_dgrad_attn_c = 17
    gemm_wgrad_attn_c = 18
    gemm_dgrad_attn_l = 19
    gemm_wgrad_attn_l = 20
    gemm_wgrad_mlp_c_n = 114
    gemm_wgrad_mlp_l_n = 116
    gemm_wgrad_attn_c_n = 118
    gemm_wgrad_attn_l_n = 120
    swiglu_bwd = 21
    bda_mlp_bwd = 22
    bda_bwd_attn = 23
    attn_bwd = 24
    ln_bwd_mlp = 25
    ln_bwd_attn = 26
    allgather_ln_mlp = 27
    allgather_ln_attn = 28
    ring_attn_fwd = 29
    ring_attn_bwd = 30
    rope = 31        # not in the reference
    rope_bwd = 32    # not in the reference


@dataclass
class LayerConfig:
    """Megatron-style GLOBAL model sizes plus the tensor-parallel degree; per-rank sizes
    are derived (the reference divides by tensor_model_parallel_size in every adapter)."""
    hidden_size: int
    num_attention_heads: int
    num_query_groups: int
    ffn_hidden_size: int
    seq_length: int
    micro_batch_size: int = 1
    tensor_model_parallel_size: int = 1
    tp_rank: int = 0
    context_parallel_size: int = 1    # > 1: seq_length is this rank's LOCAL length (zig-zag chunks cp_rank, 2cp-1-cp_rank)
    cp_rank: int = 0
    layernorm_epsilon: float = 1e-5
    rope_theta: Optional[float] = 10000.0
    params_dtype: torch.dtype = torch.bfloat16
    layernorm_bias: bool = False      # False: RMSNorm (Llama); True: LayerNorm with bias (the reference's TE call)
    comm_standin_us: float = 0.0      # > 0: every sequence-parallel stand-in also occupies its stream this long
    lockstep_blocks: bool = False     # the two strands enter every plan block together (events between the streams)
    # (forward strand's, backward strand's) communication streams: the stand-ins' delays run there, with events
    # to and from the strand's own stream, instead of on the strand's stream itself
    comm_streams: Optional[tuple] = None

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def heads_per_rank(self) -> int:
        return self.num_attention_heads // self.tensor_model_parallel_size

    @property
    def groups_per_rank(self) -> int:
        return self.num_query_groups // self.tensor_model_parallel_size

    @property
    def ffn_per_rank(self) -> int:
        return self.ffn_hidden_size // self.tensor_model_parallel_size

    @property
    def qkv_per_rank(self) -> int:
        return (self.heads_per_rank + 2 * self.groups_per_rank) * self.head_dim

    @property
    def tokens(self) -> int:
        return self.micro_batch_size * self.seq_length

    @property
    def sp_rows(self) -> int:
        return self.tokens // self.tensor_model_parallel_size

    @property
    def softmax_scale(self) -> float:
        return 1.0 / math.sqrt(self.head_dim)


def _use(t, stream):
    """Tell the caching allocator that ``t`` is consumed on ``stream``."""
    if isinstance(t, torch.Tensor) and t.is_cuda:
        t.record_stream(stream)
    return t


def _split_qkv(config: LayerConfig, qkv: torch.Tensor):
    """[T, (hq + 2 hk) d] -> q [T, hq, d], k, v [T, hk, d].  One kv group per rank: strided
    views of ``qkv``.  Several groups: contiguous copies, as the reference makes
    (dstb.py:122-125)."""
    hq, hk, d = config.heads_per_rank, config.groups_per_rank, config.head_dim
    T = qkv.shape[0]
    r = hq // hk
    if hk == 1:
        return (qkv[:, : hq * d].view(T, hq, d), qkv[:, hq * d:(hq + 1) * d].view(T, 1, d),
                qkv[:, (hq + 1) * d:].view(T, 1, d))
    g = qkv.view(T, hk, (r + 2) * d)
    q = g[:, :, : r * d].contiguous().view(T, hq, d)
    k = g[:, :, r * d:(r + 1) * d].contiguous()
    v = g[:, :, (r + 1) * d:].contiguous()
    return q, k, v


class DCFunc:
    """Per-op adapters: reshape, call the operator, return what perform_operation stores."""

    # ---- forward ----------------------------------------------------------------------
    @staticmethod
    def ln_attn(config, data, stream):
        input, ln_weight, ln_bias = data
        inputmat = input.view((-1, ln_weight.numel()))
        output, mu, rsigma, _ = pylayernorm_fwd(inputmat, ln_weight, ln_bias, config.layernorm_epsilon, 0, False,
                                                stream, profiling=False)
        return output, mu, rsigma, inputmat, input, output

    ln_mlp = ln_attn

    @staticmethod
    def gemm_attn_column(config, data, stream):
        input, weight = data
        output, _ = gemm_fwd(config, input, weight, None, "TN", False, 0, True, stream)
        return output

    @staticmethod
    def gemm_attn_linear(config, data, stream):
        input, weight = data
        input = input.view(-1, input.shape[-1])
        output, _ = gemm_fwd(config, input, weight, None, "TN", False, 0, True, stream)
        return output, input

    gemm_mlp_column = gemm_attn_column

    @staticmethod
    def gemm_mlp_linear(config, data, stream):
        input, weight = data
        input = input.view(config.tokens, -1)
        output, _ = gemm_fwd(config, input, weight, None, "TN", False, 0, True, stream)
        return output, input

    @staticmethod
    def rope(config, data, stream):
        """In place on the q and k parts of the packed projection output."""
        (qkv,) = data
        # With several kv groups q and k are not views of qkv; RoPE then runs inside fl_attn.
        if config.rope_theta is None or config.groups_per_rank != 1:
            return qkv
        q, k, _ = _split_qkv(config, qkv)
        rope_fwd(q, k, None, config.rope_theta, config.seq_length, stream, False, inplace=True)
        return qkv

    @staticmethod
    def attn(config, data, stream, apply_rope=False):
        qkv, cu_seqlens_q, cu_seqlens_kv = data
        with torch.cuda.stream(stream):
            q, k, v = _split_qkv(config, qkv)
            if apply_rope and config.rope_theta is not None:
                rope_fwd(q, k, None, config.rope_theta, config.seq_length, stream, False, inplace=True)
            out, q_p, k_p, v_p, out_p, lse, _, rng_state = pymha_varlen_fwd(
                q, k, v, cu_seqlens_q, cu_seqlens_kv, config.seq_length, config.seq_length, 0.0,
                config.softmax_scale, True, False, 0, False)
            output = out.view(config.tokens, -1)
        return output, q_p, k_p, v_p, out_p, rng_state, lse

    @staticmethod
    def ring_attn_fwd(config, data, stream):
        """One ring step (dstb.py:146-197).  ``input`` is the projection output [T, qkv] on the first step,
        afterwards the carry list of fa_cp_block_fwd.  ``visiting``: the KV chunks [2, b, 2, s/2, hk, d] that
        arrive at steps 1 .. cp-1 (already rotated by the ranks they come from).  Returns the carry list, or on
        the last step (out [T, hq d], q, kv buffers, softmax_lse, rng_states)."""
        input, cu_seqlens_q, cu_seqlens_kv, positions, visiting = data
        cp, s, b = config.context_parallel_size, config.seq_length, config.micro_batch_size
        hq, hk, d = config.heads_per_rank, config.groups_per_rank, config.head_dim
        with torch.cuda.stream(stream):
            if isinstance(input, torch.Tensor):
                if visiting is None or len(visiting) != cp - 1:
                    raise RuntimeError(f"ring attention needs the micro-batch's {cp - 1} visiting KV chunks")
                q, k, v = _split_qkv(config, input)
                if config.rope_theta is not None:
                    rope_fwd(q, k, positions, config.rope_theta, s, stream, False, inplace=True)
                own = torch.stack((k.reshape(b, 2, s // 2, hk, d), v.reshape(b, 2, s // 2, hk, d)))
                input = [q.view(b, 2, s // 2, hq, d), [own, *visiting], None, None, None, None, None, 0]
            i = input[7]
            r = fa_cp_block_fwd(input[0], cu_seqlens_q, cu_seqlens_kv, s, s, input[1], input[2], input[3], input[4],
                                input[5], input[6], i, True, RingGroup(config.cp_rank, cp), list(range(cp)), stream,
                                softmax_scale=config.softmax_scale)
            if i == cp - 1:
                out, q, _, softmax_lse, rng_states = r
                return out.view(config.tokens, -1), q, input[1], softmax_lse, rng_states
        return r[0]

    @staticmethod
    def ring_attn_bwd(config, data, stream):
        """One backward ring call (dstb.py:199-263), cp + 1 of them.  ``input`` is the gradient of the attention
        output on the first call, afterwards the state list of fa_cp_block_bwd.  The last call returns the packed
        gradient [T, qkv] of the projection output: dq, and dk / dv of this rank's OWN chunk (what the other
        ranks would add to it travels with the ring and is absent here)."""
        input, out, q, kv, softmax_lse, rng_states, cu_seqlens_q, cu_seqlens_kv, positions = data
        cp, s, b = config.context_parallel_size, config.seq_length, config.micro_batch_size
        hq, hk, d = config.heads_per_rank, config.groups_per_rank, config.head_dim
        T = config.tokens
        with torch.cuda.stream(stream):
            if isinstance(input, torch.Tensor):
                input = [input, None, None, kv, 0]
            i = input[4]
            r = fa_cp_block_bwd(input[0], out, q, input[1], None, input[2], softmax_lse, rng_states, cu_seqlens_q,
                                cu_seqlens_kv, s, s, input[3], i, True, RingGroup(config.cp_rank, cp),
                                list(range(cp)), stream, softmax_scale=config.softmax_scale)
            if i < cp:
                return r[0]
            dq, dkv = r
            dq = dq.reshape(T, hq, d)
            dk, dv = dkv[0][0].reshape(T, hk, d), dkv[0][1].reshape(T, hk, d)
            if config.rope_theta is not None:
                rope_bwd(dq, dk, positions, config.rope_theta, s, stream, False, inplace=True)
            dqkv = torch.empty((T, config.qkv_per_rank), dtype=dq.dtype, device=dq.device)
            rr = hq // hk
            torch.cat((dq.view(T, hk, rr * d), dk, dv), dim=2, out=dqkv.view(T, hk, (rr + 2) * d))
        return dqkv

    @staticmethod
    def bda_mlp(config, data, stream):
        input, residual = data
        input = input.view(config.micro_batch_size, config.seq_length // config.tensor_model_parallel_size, -1)
        output, mask, _ = bda_fwd(input, residual, stream, False, out=torch.empty_like(residual))
        return output, mask

    bda_attn = bda_mlp

    @staticmethod
    def swiglu(config, data, stream):
        (input,) = data
        input = input.view(config.micro_batch_size, config.seq_length, -1)
        output, _ = swiglu(input, stream, False)
        return output

    # ---- backward ---------------------------------------------------------------------
    @staticmethod
    def bda_attn_bwd(config, data, stream):
        grad_output, mask = data
        grad_output = grad_output.view(config.micro_batch_size, -1, grad_output.shape[-1])
        residual_bwd, output, _ = bda_bwd(grad_output, mask, None, stream, False)
        return output.view(-1, output.shape[-1]), residual_bwd

    bda_mlp_bwd = bda_attn_bwd

    @staticmethod
    def _dgrad(config, data, stream):
        grad_output, weight = data
        output, _ = dgrad_bwd(config, grad_output, weight, None, is_matmul=True, stream=stream)
        return output

    gemm_dgrad_mlp_c = gemm_dgrad_mlp_l = gemm_dgrad_attn_c = gemm_dgrad_attn_l = _dgrad

    @staticmethod
    def gemm_wgrad_attn_c(config, data, stream):
        input, grad_output, main_grad = data
        wgrad_bwd(config, grad_output, input, main_grad, is_matmul=True, stream=stream)
        return None

    gemm_wgrad_mlp_c = gemm_wgrad_attn_c

    @staticmethod
    def gemm_wgrad_attn_l(config, data, stream):
        grad_output, input, main_grad = data
        wgrad_bwd(config, grad_output, input, main_grad, is_matmul=True, stream=stream)
        return None

    gemm_wgrad_mlp_l = gemm_wgrad_attn_l

    @staticmethod
    def swiglu_bwd(config, data, stream):
        swiglu_input, grad_output = data
        swiglu_input = swiglu_input.view(-1, swiglu_input.shape[-1])
        dgrad, _ = swiglu_back(grad_output, swiglu_input, None, stream, profiling=False)
        return dgrad

    @staticmethod
    def attn_bwd(config, data, stream, apply_rope=False):
        grad_output, q, k, v, out, lse, cu_seqlens_q, cu_seqlens_kv, rng_state = data
        hq, hk, d = config.heads_per_rank, config.groups_per_rank, config.head_dim
        T = grad_output.shape[0]
        with torch.cuda.stream(stream):
            dout = grad_output.view(T, hq, d)
            dqkv = torch.empty((T, config.qkv_per_rank), dtype=q.dtype, device=q.device)
            if hk == 1:
                dq, dk, dv = _split_qkv(config, dqkv)      # views: the kernels write the packed gradient directly
            else:
                dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
            _attn_bwd_raw(dout, q, k, v, out, lse, dq, dk, dv, None, cu_seqlens_q, cu_seqlens_kv, config.seq_length,
                          config.seq_length, config.softmax_scale, True, stream.cuda_stream)
            if apply_rope and config.rope_theta is not None:
                rope_bwd(dq, dk, None, config.rope_theta, config.seq_length, stream, False, inplace=True)
            if hk != 1:
                r = hq // hk
                torch.cat((dq.view(T, hk, r * d), dk, dv), dim=2, out=dqkv.view(T, hk, (r + 2) * d))
        return dqkv

    @staticmethod
    def rope_bwd(config, data, stream):
        (dqkv,) = data
        if config.rope_theta is None or config.groups_per_rank != 1:   # several groups: done inside attn_bwd
            return dqkv
        dq, dk, _ = _split_qkv(config, dqkv)
        rope_bwd(dq, dk, None, config.rope_theta, config.seq_length, stream, False, inplace=True)
        return dqkv

    @staticmethod
    def ln_mlp_bwd(config, data, stream):
        output, ln_input, ln_mu, ln_rsigma, ln_weight, ln_bias, residual, w_main_grad, b_main_grad = data
        dgrad, _, _, _ = pylayernorm_bwd(output, ln_input, ln_mu, ln_rsigma, ln_weight, 0, False, stream, False,
                                         add_to_dgrad=residual, dgamma_out=w_main_grad,
                                         dbeta_out=b_main_grad if ln_mu is not None else None)
        return dgrad

    @staticmethod
    def ln_attn_bwd(config, data, stream):
        dgrad = DCFunc.ln_mlp_bwd(config, data, stream)
        return dgrad.view(config.micro_batch_size, -1, dgrad.shape[-1])

    # ---- sequence-parallel stand-ins (one GPU: no collective is issued) ---------------
    @staticmethod
    def _comm_delay(config, stream, bwd_strand=False):
        """With ``comm_standin_us`` set, a stand-in also keeps its stream busy for that long (a one-wavefront
        kernel that touches no memory): the duration of the collective it replaces, for schedule experiments."""
        us = getattr(config, "comm_standin_us", 0.0)
        if us > 0:
            st = stream if stream is not None else torch.cuda.current_stream()
            comm = getattr(config, "comm_streams", None)
            if comm is None:
                _lib.check(_lib.load().dh_delay(int(us * 1000), st.cuda_stream))
                return
            cs = comm[1] if bwd_strand else comm[0]
            posted, done = torch.cuda.Event(), torch.cuda.Event()
            posted.record(st)
            cs.wait_event(posted)
            _lib.check(_lib.load().dh_delay(int(us * 1000), cs.cuda_stream))
            done.record(cs)
            st.wait_event(done)

    @staticmethod
    def allgather(config, data, stream, bwd_strand=False):
        """(out, handle).  ``peer`` holds the other ranks' rows for this micro-batch."""
        input, peer = data
        tp = config.tensor_model_parallel_size
        if tp == 1:
            return input.view(-1, input.shape[-1]), None
        DCFunc._comm_delay(config, stream, bwd_strand)
        if peer is None:
            raise RuntimeError("sequence-parallel gather stand-in needs the micro-batch's peer buffer")
        rows = input.numel() // input.shape[-1]
        dst = peer[config.tp_rank * rows:(config.tp_rank + 1) * rows]
        src = input.view(rows, -1)
        assert dst.is_contiguous() and src.is_contiguous() and dst.dtype == src.dtype and dst.shape == src.shape
        st = stream if stream is not None else torch.cuda.current_stream()
        _lib.check(_lib.load().dh_copy_bytes(src.data_ptr(), dst.data_ptr(), src.numel() * src.element_size(),
                                             st.cuda_stream))
        return peer, None

    @staticmethod
    def reduce_scatter(config, data, stream, bwd_strand=False):
        (input,) = data
        tp = config.tensor_model_parallel_size
        if tp == 1:
            return input, None
        DCFunc._comm_delay(config, stream, bwd_strand)
        rows = input.shape[0] // tp
        return input[config.tp_rank * rows:(config.tp_rank + 1) * rows], None


# activation keys popped (freed) per op id after it ran; mirrors dstb.py:506-656
_FREE_AFTER = {
    8: ["ln_mlp_residual"], 9: ["ln_attn_residual"],
    14: ["swiglu_dgrad", "gemm_mlp_c_input"], 16: ["linear_mlp_input"], 18: ["gemm_attn_c_input"],
    20: ["linear_attn_input"], 21: ["swiglu_input"], 22: ["mlp_mask"], 23: ["attn_mask"],
    24: ["q_padded", "k_padded", "v_padded", "out_padded", "softmax_lse", "rng_state"],
    25: ["ln_mlp_input", "mlp_mu", "mlp_rsigma", "mlp_residual_bwd"],
    26: ["ln_attn_input", "attn_mu", "attn_rsigma", "attn_residual_bwd"],
}

_WGRAD_PLACEHOLDER = {14: "gemm_wgrad_mlp_c_n", 16: "gemm_wgrad_mlp_l_n", 18: "gemm_wgrad_attn_c_n",
                      20: "gemm_wgrad_attn_l_n"}
_PLACEHOLDER_ID = {114: "gemm_wgrad_mlp_c_n", 116: "gemm_wgrad_mlp_l_n", 118: "gemm_wgrad_attn_c_n",
                   120: "gemm_wgrad_attn_l_n"}
# name of the peer buffer each stand-in gather uses, keyed by plan op name
_PEER_KEY = {"allgather_attn": "sp_peer_attn", "allgather_mlp": "sp_peer_mlp",
             "allgather_mlp_bwd": "sp_peer_mlp_bwd", "allgather_attn_bwd": "sp_peer_attn_bwd"}


class DCoperation:
    """Dispatch one op id: fetch its inputs (previous op's output, weights, saved
    activations), run the adapter, save / free activations (dstb.py:427-660)."""

    @staticmethod
    def perform_operation(dcfunc, operation, config, weight, activation_dict, **kwargs):
        stream = kwargs["stream"]
        x = kwargs.get("output")
        name = kwargs.get("name")
        movable = kwargs.get("movable", ())
        act = activation_dict
        op = operation.value if isinstance(operation, FuncChoice) else int(operation)
        g = lambda key: _use(act[key], stream)
        output = None

        if op in (1, 2):
            p = "attn" if op == 1 else "mlp"
            fn = dcfunc.ln_attn if op == 1 else dcfunc.ln_mlp
            output, act[f"{p}_mu"], act[f"{p}_rsigma"], act[f"ln_{p}_input"], act[f"ln_{p}_residual"], _ = fn(
                config, (x, weight[f"ln_{p}_weight"], weight.get(f"ln_{p}_bias")), stream)
        elif op == 3:
            act["gemm_attn_c_input"] = x
            output = dcfunc.gemm_attn_column(config, (x, weight["column_attn_weight"]), stream)
        elif op == 31:
            output = dcfunc.rope(config, (x,), stream)
        elif op == 7:
            (output, act["q_padded"], act["k_padded"], act["v_padded"], act["out_padded"], act["rng_state"],
             act["softmax_lse"]) = dcfunc.attn(config, (x, weight["cu_seqlens_q"], weight["cu_seqlens_kv"]), stream,
                                               apply_rope=config.groups_per_rank != 1)
        elif op == 4:
            output, act["linear_attn_input"] = dcfunc.gemm_attn_linear(config, (x, weight["linear_attn_weight"]), stream)
        elif op == 5:
            act["gemm_mlp_c_input"] = x
            output = dcfunc.gemm_mlp_column(config, (x, weight["column_mlp_weight"]), stream)
        elif op == 6:
            output, act["linear_mlp_input"] = dcfunc.gemm_mlp_linear(config, (x, weight["linear_mlp_weight"]), stream)
        elif op == 8:
            output, act["mlp_mask"] = dcfunc.bda_mlp(config, (x, g("ln_mlp_residual")), stream)
        elif op == 9:
            output, act["attn_mask"] = dcfunc.bda_attn(config, (x, g("ln_attn_residual")), stream)
        elif op == 10:
            output = dcfunc.reduce_scatter(config, (x,), stream, bwd_strand=bool(name) and name.endswith("_bwd"))
        elif op == 11:
            peer = act.get(_PEER_KEY.get(name, ""))
            output = dcfunc.allgather(config, (x, _use(peer, stream)), stream,
                                      bwd_strand=bool(name) and name.endswith("_bwd"))
        elif op == 12:
            output = dcfunc.swiglu(config, (x,), stream)
            act["swiglu_input"] = x
        elif op in (13, 15, 17, 19):
            wkey = {13: "column_mlp_weight", 15: "linear_mlp_weight", 17: "column_attn_weight",
                    19: "linear_attn_weight"}[op]
            output = dcfunc._dgrad(config, (x, weight[wkey]), stream)
        elif op in (14, 18):
            # (saved GEMM input, incoming gradient, main_grad)
            if op == 14:
                args = (g("gemm_mlp_c_input"), g("swiglu_dgrad"), weight["column_mlp_weight"].main_grad)
                fn = dcfunc.gemm_wgrad_mlp_c
            else:
                args = (g("gemm_attn_c_input"), x, weight["column_attn_weight"].main_grad)
                fn = dcfunc.gemm_wgrad_attn_c
            if _WGRAD_PLACEHOLDER[op] in movable:
                act.setdefault("_parked", {})[_WGRAD_PLACEHOLDER[op]] = (fn, (config, args, stream))
            else:
                fn(config, args, stream)
        elif op in (16, 20):
            key, wkey = ("linear_mlp_input", "linear_mlp_weight") if op == 16 else ("linear_attn_input", "linear_attn_weight")
            args = (x, g(key), weight[wkey].main_grad)
            fn = dcfunc.gemm_wgrad_mlp_l if op == 16 else dcfunc.gemm_wgrad_attn_l
            if _WGRAD_PLACEHOLDER[op] in movable:
                act.setdefault("_parked", {})[_WGRAD_PLACEHOLDER[op]] = (fn, (config, args, stream))
            else:
                fn(config, args, stream)
        elif op in _PLACEHOLDER_ID:
            parked = act.get("_parked", {}).pop(_PLACEHOLDER_ID[op], None)
            if parked is not None:
                fn, (cfg, args, _) = parked
                fn(cfg, args, stream)
        elif op == 21:
            output = dcfunc.swiglu_bwd(config, (g("swiglu_input"), x), stream)
            act["swiglu_dgrad"] = output
        elif op == 22:
            output, act["mlp_residual_bwd"] = dcfunc.bda_mlp_bwd(config, (x, act.get("mlp_mask")), stream)
        elif op == 23:
            output, act["attn_residual_bwd"] = dcfunc.bda_attn_bwd(config, (x, act.get("attn_mask")), stream)
        elif op == 24:
            output = dcfunc.attn_bwd(config, (x, g("q_padded"), g("k_padded"), g("v_padded"), g("out_padded"),
                                              g("softmax_lse"), weight["cu_seqlens_q"], weight["cu_seqlens_kv"],
                                              act.get("rng_state")), stream,
                                     apply_rope=config.groups_per_rank != 1)
        elif op == 32:
            output = dcfunc.rope_bwd(config, (x,), stream)
        elif op == 29:
            last = (0 if isinstance(x, torch.Tensor) else x[7]) == config.context_parallel_size - 1
            visiting = act.get("cp_kv_chunks")
            if visiting is not None:
                for t in visiting:
                    _use(t, stream)
            output = dcfunc.ring_attn_fwd(config, (x, weight["cu_seqlens_q"], weight["cu_seqlens_kv"],
                                                   weight.get("rope_positions"), visiting), stream)
            if last:
                output, act["q"], act["kv"], act["softmax_lse"], act["rng_states"] = output
                act["out"] = output
        elif op == 30:
            last = (0 if isinstance(x, torch.Tensor) else x[4]) == config.context_parallel_size
            for t in act["kv"]:
                _use(t, stream)
            output = dcfunc.ring_attn_bwd(config, (x, g("out"), g("q"), act["kv"], g("softmax_lse"), act.get("rng_states"),
                                                   weight["cu_seqlens_q"], weight["cu_seqlens_kv"],
                                                   weight.get("rope_positions")), stream)
            if last:
                for key in ("out", "q", "kv", "softmax_lse", "rng_states"):
                    act.pop(key, None)
                act["attn_dgrad"] = output
        elif op in (25, 26):
            p = "mlp" if op == 25 else "attn"
            lw, lb = weight[f"ln_{p}_weight"], weight.get(f"ln_{p}_bias")
            mu = act.get(f"{p}_mu")
            data = (x, g(f"ln_{p}_input"), _use(mu, stream), g(f"{p}_rsigma"), lw, lb, g(f"{p}_residual_bwd"),
                    lw.main_grad, lb.main_grad if lb is not None else None)
            output = (dcfunc.ln_mlp_bwd if op == 25 else dcfunc.ln_attn_bwd)(config, data, stream)
        else:
            raise ValueError(f"operation {op} is not part of the single-GPU decoder-layer path")

        if op == 18:
            act.pop("attn_dgrad", None)          # kept by the last ring call for the qkv weight gradient
        for key in _FREE_AFTER.get(op, ()):
            act.pop(key, None)
        return output


class DCOP:
    """A node of the op graph (dstb.py:662-690)."""

    def __init__(self, pre_op, stream, num, is_first_mb, is_comm=0, name=None):
        self.pre = pre_op
        self.stream = stream
        self.op_num = num
        self.is_first_mb = is_first_mb
        self.is_comm = is_comm      # 0 compute, 1 forward-strand comm, 2 backward-strand comm
        self.name = name
        self.next_op: list = []
        self.handle = None
        self.output = None

    def __str__(self) -> str:
        return self.name or FuncChoice(self.op_num).name

    def set_next_op(self, next_op): self.next_op.append(next_op)
    def set_handle(self, handle): self.handle = handle
    def get_handle(self): return self.handle
    def set_output(self, output): self.output = output
    def get_op_num(self): return self.op_num
    def get_output(self): return self.output
    def get_next_op(self): return self.next_op


class DCBlock:
    def __init__(self, stream1_op: Optional[List[DCOP]], stream2_op: Optional[List[DCOP]],
                 stream3_op: Optional[List[DCOP]]):
        self.stream1_op = stream1_op
        self.stream2_op = stream2_op
        self.stream3_op = stream3_op


# (name, op id, strand: 1 fwd / 2 bwd, is_comm, predecessor)
_GRAPH = [
    ("ln_attn", 1, 1, 0, None), ("allgather_attn", 11, 1, 1, "ln_attn"), ("gemm_attn_c", 3, 1, 0, "allgather_attn"),
    ("rope", 31, 1, 0, "gemm_attn_c"), ("fl_attn", 7, 1, 0, "rope"), ("gemm_attn_l", 4, 1, 0, "fl_attn"),
    ("reduce_scatter_attn", 10, 1, 1, "gemm_attn_l"), ("bda_attn", 9, 1, 0, "reduce_scatter_attn"),
    ("ln_mlp", 2, 1, 0, "bda_attn"), ("allgather_mlp", 11, 1, 1, "ln_mlp"), ("gemm_mlp_c", 5, 1, 0, "allgather_mlp"),
    ("swiglu_mlp", 12, 1, 0, "gemm_mlp_c"), ("gemm_mlp_l", 6, 1, 0, "swiglu_mlp"),
    ("reduce_scatter_mlp", 10, 1, 1, "gemm_mlp_l"), ("bda_mlp", 8, 1, 0, "reduce_scatter_mlp"),
    ("bda_mlp_bwd", 22, 2, 0, None), ("allgather_mlp_bwd", 11, 2, 2, "bda_mlp_bwd"),
    ("gemm_dgrad_mlp_l", 15, 2, 0, "allgather_mlp_bwd"), ("gemm_wgrad_mlp_l", 16, 2, 0, "allgather_mlp_bwd"),
    ("swiglu_bwd", 21, 2, 0, "gemm_dgrad_mlp_l"), ("gemm_dgrad_mlp_c", 13, 2, 0, "swiglu_bwd"),
    ("gemm_wgrad_mlp_c", 14, 2, 0, "swiglu_bwd"), ("reduce_scatter_mlp_c_bwd", 10, 2, 2, "gemm_dgrad_mlp_c"),
    ("ln_mlp_bwd", 25, 2, 0, "reduce_scatter_mlp_c_bwd"), ("bda_attn_bwd", 23, 2, 0, "ln_mlp_bwd"),
    ("allgather_attn_bwd", 11, 2, 2, "bda_attn_bwd"), ("gemm_dgrad_attn_l", 19, 2, 0, "allgather_attn_bwd"),
    ("gemm_wgrad_attn_l", 20, 2, 0, "allgather_attn_bwd"), ("attn_bwd", 24, 2, 0, "gemm_dgrad_attn_l"),
    ("rope_bwd", 32, 2, 0, "attn_bwd"), ("gemm_dgrad_attn_c", 17, 2, 0, "rope_bwd"),
    ("gemm_wgrad_attn_c", 18, 2, 0, "rope_bwd"), ("reduce_scatter_attn_c_bwd", 10, 2, 2, "gemm_dgrad_attn_c"),
    ("ln_attn_bwd", 26, 2, 0, "reduce_scatter_attn_c_bwd"),
    ("gemm_wgrad_mlp_c_n", 114, 2, 0, None), ("gemm_wgrad_mlp_l_n", 116, 2, 0, None),
    ("gemm_wgrad_attn_c_n", 118, 2, 0, None), ("gemm_wgrad_attn_l_n", 120, 2, 0, None),
]

# Built-in plans (dstb.py:1043-1060, 1080-1093, 1115-1129), in the plan-file schema.
DEFAULT_PLAN = {
    "DCBlocks": [
        [["ln_attn"], "None", "None"],
        ["None", ["bda_mlp_bwd"], ["allgather_attn"]],
        [["gemm_attn_c", "fl_attn"], "None", ["allgather_mlp_bwd"]],
        [["gemm_attn_l"], "None", "None"],
        ["None", ["gemm_dgrad_mlp_l", "gemm_wgrad_mlp_l"], ["reduce_scatter_attn"]],
        ["None", ["swiglu_bwd"], "None"],
        ["None", ["gemm_dgrad_mlp_c"], "None"],
        ["None", ["gemm_wgrad_mlp_c"], ["reduce_scatter_mlp_c_bwd"]],
        [["bda_attn", "ln_mlp"], "None", "None"],
        ["None", ["ln_mlp_bwd", "bda_attn_bwd"], ["allgather_mlp"]],
        [["gemm_mlp_c"], "None", ["allgather_attn_bwd"]],
        [["swiglu_mlp", "gemm_mlp_l"], "None", "None"],
        ["None", ["gemm_dgrad_attn_l", "gemm_wgrad_attn_l", "attn_bwd"], ["reduce_scatter_mlp"]],
        [["bda_mlp"], "None", "None"],
        ["None", ["gemm_dgrad_attn_c"], "None"],
        ["None", ["gemm_wgrad_attn_c"], ["reduce_scatter_attn_c_bwd"]],
        ["None", ["ln_attn_bwd"], "None"],
    ],
    "fwd_only": [
        [["ln_attn"], "None", "None"], ["None", "None", ["allgather_attn"]],
        [["gemm_attn_c", "fl_attn"], "None", "None"], [["gemm_attn_l"], "None", "None"],
        ["None", "None", ["reduce_scatter_attn"]], [["bda_attn", "ln_mlp"], "None", "None"],
        ["None", "None", ["allgather_mlp"]], [["gemm_mlp_c"], "None", "None"],
        [["swiglu_mlp", "gemm_mlp_l"], "None", "None"], ["None", "None", ["reduce_scatter_mlp"]],
        [["bda_mlp"], "None", "None"],
    ],
    "bwd_only": [
        ["None", ["bda_mlp_bwd"], "None"], ["None", "None", ["allgather_mlp_bwd"]],
        ["None", ["gemm_dgrad_mlp_l", "gemm_wgrad_mlp_l"], "None"], ["None", ["swiglu_bwd"], "None"],
        ["None", ["gemm_dgrad_mlp_c"], "None"], ["None", ["gemm_wgrad_mlp_c"], ["reduce_scatter_mlp_c_bwd"]],
        ["None", ["ln_mlp_bwd", "bda_attn_bwd"], "None"], ["None", "None", ["allgather_attn_bwd"]],
        ["None", ["gemm_dgrad_attn_l", "gemm_wgrad_attn_l", "attn_bwd"], "None"],
        ["None", ["gemm_dgrad_attn_c"], "None"], ["None", ["gemm_wgrad_attn_c"], ["reduce_scatter_attn_c_bwd"]],
        ["None", ["ln_attn_bwd"], "None"],
    ],
}


class Plan:
    """The three block lists of a plan plus per-plan state (the reference keeps the list of
    deferred wgrad ops in a module global that grows on every call, dstb.py:16,931-939)."""

    def __init__(self, dcblocks, fwd_only, bwd_only, movable, ops):
        self.dcblocks, self.fwd_only, self.bwd_only = dcblocks, fwd_only, bwd_only
        self.movable = frozenset(movable)
        self.ops = ops          # name -> DCOP

    def __iter__(self):         # so that ``dcblocks, fwd_only, bwd_only = init_DCBlocks(...)`` works
        return iter((self.dcblocks, self.fwd_only, self.bwd_only))


def _names(entry):
    if entry is None or entry == "None":
        return None
    if isinstance(entry, str):
        return [entry]
    return [e for e in entry if e != "None"] or None


def ring_op_names(cp: int):
    """Plan names of the ring steps: cp forward steps, cp + 1 backward calls (the reference writes them out for
    cp = 2: cp_attn_block_fwd_1/2, cp_attn_block_bwd_1/2/3, dstb.py:711-722,801-817)."""
    return ([f"cp_attn_block_fwd_{i}" for i in range(1, cp + 1)],
            [f"cp_attn_block_bwd_{i}" for i in range(1, cp + 2)])


def _graph(cp: int):
    """The op graph as (name, op id, strand, is_comm, predecessor) rows; with cp > 1 the ring steps stand where
    rope + fl_attn and attn_bwd + rope_bwd stand otherwise (RoPE then runs inside the first / last ring call)."""
    if cp <= 1:
        return _GRAPH
    fwd, bwd = ring_op_names(cp)
    rows = []
    for row in _GRAPH:
        name, num, strand, is_comm, pre = row
        if name in ("rope", "rope_bwd"):
            continue
        if name == "fl_attn":
            prev = "gemm_attn_c"
            for n in fwd:
                rows.append((n, 29, 1, 0, prev))
                prev = n
            continue
        if name == "attn_bwd":
            prev = "gemm_dgrad_attn_l"
            for n in bwd:
                rows.append((n, 30, 2, 0, prev))
                prev = n
            continue
        if pre == "fl_attn":
            pre = fwd[-1]
        elif pre == "rope_bwd":
            pre = bwd[-1]
        rows.append((name, num, strand, is_comm, pre))
    return rows


def _ring_names_for(blocks_json, cp):
    """A plan written without context parallelism, used with cp > 1: fl_attn / attn_bwd become the ring steps
    (in the same column), the RoPE ops disappear."""
    fwd, bwd = ring_op_names(cp)
    named = {n for blk in blocks_json for col in blk for n in (_names(col) or [])}
    has_ring = any(n.startswith("cp_attn_block_") for n in named)
    out = []
    for blk in blocks_json:
        cols = []
        for col in blk:
            names = _names(col)
            if names is not None:
                new = []
                for n in names:
                    if n in ("rope", "rope_bwd"):
                        continue
                    if n == "fl_attn" and not has_ring:
                        new.extend(fwd)
                    elif n == "attn_bwd" and not has_ring:
                        new.extend(bwd)
                    else:
                        new.append(n)
                names = new or None
            cols.append(names)
        out.append(cols)
    return out


def _insert_rope(blocks_json):
    """Plans written for the reference never name the RoPE ops: put ``rope`` right before
    ``fl_attn`` and ``rope_bwd`` right after ``attn_bwd``, in the same column."""
    named = {n for blk in blocks_json for col in blk for n in (_names(col) or [])}
    out = []
    for blk in blocks_json:
        cols = []
        for col in blk:
            names = _names(col)
            if names is not None:
                new = []
                for n in names:
                    if n == "fl_attn" and "rope" not in named:
                        new.append("rope")
                    new.append(n)
                    if n == "attn_bwd" and "rope_bwd" not in named:
                        new.append("rope_bwd")
                names = new
            cols.append(names)
        out.append(cols)
    return out


def init_DCBlocks(config=None, stream1=None, stream2=None, context_parallel_size: int = 1) -> Plan:
    """Build the op graph and map a plan onto it.  ``config``: path of a plan JSON, a dict in
    the same schema, or None for the built-in plans.  Schema (search/search.py:180-244):
    {"DCBlocks": [[stream1, stream2, stream3], ...], "fwd_only": [...], "bwd_only": [...]},
    each column a list of op names, one name, or "None"; missing sections use the built-ins.
    ``context_parallel_size`` > 1 builds the graph with the ring steps (the reference reads it
    from Megatron's global arguments, dstb.py:709)."""
    ops = {}
    cp = int(context_parallel_size)
    for name, num, strand, is_comm, pre in _graph(cp):
        node = DCOP(ops.get(pre), stream1 if strand == 1 else stream2, num, name == "ln_attn", is_comm, name)
        node.strand = strand
        if pre is not None:
            ops[pre].set_next_op(node)
        ops[name] = node
    if isinstance(config, str):
        with open(config, "r") as f:
            data = json.load(f)
    else:
        data = config or {}
    if "DCBlocks" not in data and config is not None:
        raise KeyError("plan has no 'DCBlocks' section")
    movable = set()

    def build(section):
        blocks = []
        raw = data.get(section) or DEFAULT_PLAN[section]
        for blk in (_insert_rope(raw) if cp <= 1 else _ring_names_for(raw, cp)):
            if len(blk) != 3:
                raise ValueError(f"a plan block has 3 columns [stream1, stream2, stream3], got {blk!r}")
            cols = []
            for ci, names in enumerate(blk):
                if names is None:
                    cols.append(None)
                    continue
                col = []
                for n in names:
                    if n not in ops:
                        raise KeyError(f"unknown op name in plan: {n!r}")
                    if n.endswith("_n") and ci == 1:
                        movable.add(n)
                    col.append(ops[n])
                cols.append(col)
            blocks.append(DCBlock(*cols))
        return blocks

    return Plan(build("DCBlocks"), build("fwd_only"), build("bwd_only"), movable, ops)


def _run_column(col, dcoperation, config, weight, act, first_input, stream_of, result, movable):
    for now_op in col:
        src = now_op.get_output()
        inp = first_input if src is None else src
        st = stream_of(now_op)
        output = dcoperation.perform_operation(DCFunc, now_op.get_op_num(), config, weight, act, output=inp, stream=st,
                                               name=now_op.name, movable=movable)
        handle = None
        if now_op.is_comm:
            output, handle = output
        now_op.set_output(None)
        nxt = now_op.get_next_op()
        if output is not None and len(nxt) == 0:
            result[0] = output
        for nop in nxt:
            nop.set_output(output)
            nop.set_handle(handle)


def exec(config, dcoperation, fwd_weight, bwd_weight, input, grad_output, dcblocks: List[DCBlock], stream1, stream2,
         activation_dict, new_activation_dict, movable=()):
    """Walk the blocks of a plan (dstb.py:1133-1281): forward ops of the NEW micro-batch on
    ``stream1`` (reading/writing ``new_activation_dict`` with ``fwd_weight``), backward ops
    of the PREVIOUS micro-batch on ``stream2`` (``activation_dict``, ``bwd_weight``), stand-in
    comm ops on the stream of the strand they belong to.  Returns (fwd_result, bwd_result).

    Nothing here waits for the device.  ``activation_dict['_ready']`` (an event recorded
    when that micro-batch's forward was fully issued) is waited on by ``stream2`` first;
    when this call issues a forward, ``new_activation_dict['_ready']`` is recorded on
    ``stream1`` at the end."""
    fwd_res, bwd_res = [None], [None]
    if activation_dict is not None and stream2 is not None:
        ev = activation_dict.get("_ready")
        if ev is not None:
            stream2.wait_event(ev)
    ran_fwd = False

    def stream_of(op):
        return stream1 if getattr(op, "strand", 1) == 1 else stream2

    lockstep = (getattr(config, "lockstep_blocks", False) and stream1 is not None and stream2 is not None
                and stream1 != stream2)
    for now_block in dcblocks:
        if lockstep:
            # both strands enter a block together (device-side events, no host wait): keeps the block's pairing,
            # which matters when the stand-in collectives have a duration to hide; without it the forward strand
            # simply runs ahead
            e1, e2 = torch.cuda.Event(), torch.cuda.Event()
            e1.record(stream1)
            e2.record(stream2)
            stream1.wait_event(e2)
            stream2.wait_event(e1)
        fwd_comm_first = False
        if now_block.stream3_op is not None:
            for now_op in now_block.stream3_op:
                if now_op.is_comm == 1:
                    fwd_comm_first = True
                    _run_column([now_op], dcoperation, config, fwd_weight, new_activation_dict, input, stream_of,
                                fwd_res, movable)
                    ran_fwd = True
                else:
                    _run_column([now_op], dcoperation, config, bwd_weight, activation_dict, grad_output, stream_of,
                                bwd_res, movable)
        # The strand whose communication was just posted goes second (dstb.py:1174-1264).
        order = (2, 1) if fwd_comm_first else (1, 2)
        for strand in order:
            if strand == 1 and now_block.stream1_op is not None:
                _run_column(now_block.stream1_op, dcoperation, config, fwd_weight, new_activation_dict, input, stream_of,
                            fwd_res, movable)
                ran_fwd = True
            if strand == 2 and now_block.stream2_op is not None:
                _run_column(now_block.stream2_op, dcoperation, config, bwd_weight, activation_dict, grad_output,
                            stream_of, bwd_res, movable)
    # deferred wgrads that no placeholder op picked up run at the end (dstb.py:1268-1279)
    if activation_dict is not None and activation_dict.get("_parked"):
        for key in list(activation_dict["_parked"]):
            fn, (cfg, args, st) = activation_dict["_parked"].pop(key)
            fn(cfg, args, st)
    if ran_fwd and new_activation_dict is not None and stream1 is not None:
        ev = torch.cuda.Event()
        ev.record(stream1)
        new_activation_dict["_ready"] = ev
    return fwd_res[0], bwd_res[0]


exec_plan = exec
