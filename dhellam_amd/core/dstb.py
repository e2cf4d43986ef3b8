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
from ..common.global_variables import GLOBAL_VARIABLES
from .._Clib import (WGRAD_TRANSPOSE_GRAD_MIN_K, WGRAD_TRANSPOSE_MIN_ELEMS, keep_transposed, pymha_varlen_bwd,
                      pymha_varlen_fwd, _attn_bwd_raw)
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
    # what occupies the stream: "kernel" = a one-wavefront delay kernel launched per collective (it has to find a free
    # wavefront slot next to whatever else runs, and a kernel launched beside a GEMM that owns every compute unit
    # starts only when that GEMM has placed its last workgroup), "proxy" = a request to the resident communication
    # proxy (one kernel per step with a wavefront per strand, reached through stream writes and stream waits:
    # ``common/comm_proxy.py``; ``comm_proxy`` below must hold it -- ``LayerRunner`` sets it up), "host" = a host
    # function of the stream (a transfer carried by a copy engine or a network adapter: needs no compute unit)
    comm_standin_engine: str = "kernel"
    comm_proxy: Optional[object] = None
    lockstep_blocks: bool = False     # the two strands enter every plan block together (events between the streams)
    # (forward strand's, backward strand's) communication streams: the stand-ins' delays run there, with events
    # to and from the strand's own stream, instead of on the strand's stream itself
    comm_streams: Optional[tuple] = None
    fuse_adjacent: bool = True        # ops a plan lists next to each other run as one kernel where one exists (bda_attn + ln_mlp)
    gather_in_place: bool = True      # the op in front of a sequence-parallel all-gather writes straight into its rows of the gathered buffer
    resident_weight_transposes: bool = True   # projection weights are kept as W and W^T: the data-gradient GEMMs then run in the forward's layout

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
        kept = getattr(t, "_dh_rows_transposed", None)     # the transpose its producer left on it is consumed there too
        if kept is not None:
            kept[1].record_stream(stream)
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
    def ln_attn(config, data, stream, out=None):
        """``out``: where the result goes when it is not a new tensor (the rank's rows of the buffer that the
        sequence-parallel all-gather after this op fills, so that the gather has nothing left to copy)."""
        input, ln_weight, ln_bias = data
        inputmat = input.view((-1, ln_weight.numel()))
        output, mu, rsigma, _ = pylayernorm_fwd(inputmat, ln_weight, ln_bias, config.layernorm_epsilon, 0, False,
                                                stream, profiling=False, ln_out=out)
        return output, mu, rsigma, inputmat, input, output

    ln_mlp = ln_attn

    @staticmethod
    def bda_attn_ln_mlp(config, data, stream, out=None):
        """``bda_attn`` and ``ln_mlp`` (dstb.py:273-277, 73-78), adjacent in the layer, in one kernel: the residual
        sum is written once and normalised from registers.  Returns (ln output, mu, rsigma, norm input as a
        matrix, the residual sum in the layer's [b, s/tp, h] shape)."""
        input, residual, ln_weight, ln_bias = data
        input = input.view(config.micro_batch_size, config.seq_length // config.tensor_model_parallel_size, -1)
        output, mu, rsigma, _, x2 = pylayernorm_fwd(input, ln_weight, ln_bias, config.layernorm_epsilon, 0, False,
                                                    stream, profiling=False, residual=residual, ln_out=out)
        x2 = x2.view(input.shape)
        return output.view(-1, ln_weight.numel()), mu, rsigma, x2.view(-1, ln_weight.numel()), x2

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
        kept = getattr(input, "_dh_rows_transposed", None)
        input = input.view(config.tokens, -1)
        if kept is not None:        # the transpose its producer wrote stays with the saved view (views share the version)
            input._dh_rows_transposed = kept
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
        # the weight-gradient product of the row projection behind the activation takes this result transposed when
        # the projection has fewer inputs than outputs (``_Clib.wgrad_layout``): the kernel then writes it alongside
        f = input.shape[-1] // 2
        want_t = f < config.hidden_size and config.tokens * f >= WGRAD_TRANSPOSE_MIN_ELEMS
        output, _ = swiglu(input, stream, False, with_transposed=want_t)
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
        # the weight-gradient product of the column projection wants this gradient transposed when the layer is
        # wide enough for that layout to pay (``_Clib.wgrad_layout``): the kernel then writes it alongside
        rows, n2 = swiglu_input.shape
        want_t = (config.hidden_size >= WGRAD_TRANSPOSE_GRAD_MIN_K and rows * n2 >= WGRAD_TRANSPOSE_MIN_ELEMS
                  and config.hidden_size >= n2)     # (fewer inputs than outputs: the input is the operand transposed)
        dgrad, _ = swiglu_back(grad_output, swiglu_input, None, stream, profiling=False, with_transposed=want_t)
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
    def ln_mlp_bwd(config, data, stream, out=None):
        output, ln_input, ln_mu, ln_rsigma, ln_weight, ln_bias, residual, w_main_grad, b_main_grad = data
        dgrad, _, _, _ = pylayernorm_bwd(output, ln_input, ln_mu, ln_rsigma, ln_weight, 0, False, stream, False,
                                         add_to_dgrad=residual, dgamma_out=w_main_grad,
                                         dbeta_out=b_main_grad if ln_mu is not None else None, dgrad_out=out)
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
            engine = getattr(config, "comm_standin_engine", "kernel")
            if engine == "proxy":
                proxy = getattr(config, "comm_proxy", None)
                if proxy is None or not proxy.running:
                    raise RuntimeError("comm_standin_engine='proxy' needs a launched CommProxy in config.comm_proxy")
                proxy.collective(1 if bwd_strand else 0, st)
                return
            delay = _lib.load().dh_host_delay if engine == "host" else _lib.load().dh_delay
            if comm is None:
                _lib.check(delay(int(us * 1000), st.cuda_stream))
                return
            cs = comm[1] if bwd_strand else comm[0]
            posted, done = torch.cuda.Event(), torch.cuda.Event()
            posted.record(st)
            cs.wait_event(posted)
            _lib.check(delay(int(us * 1000), cs.cuda_stream))
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
        if src.data_ptr() != dst.data_ptr():        # else the producer wrote the rows in place (an in-place gather)
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


class _Ctx:
    """What one dispatch hands to an op handler."""
    __slots__ = ("dcfunc", "op", "config", "weight", "act", "x", "stream", "name", "movable")

    def __init__(self, dcfunc, op, config, weight, act, x, stream, name, movable):
        self.dcfunc, self.op, self.config, self.weight, self.act = dcfunc, op, config, weight, act
        self.x, self.stream, self.name, self.movable = x, stream, name, movable

    def g(self, key):
        """A saved activation, registered with the stream that is about to read it."""
        return _use(self.act[key], self.stream)


def _gather_slot(c, gather_name):
    """This rank's rows of the buffer that the stand-in all-gather ``gather_name`` fills, or None: the op in front
    of the gather writes its result there, as the producer of an in-place all-gather does."""
    cfg = c.config
    tp = cfg.tensor_model_parallel_size
    peer = c.act.get(_PEER_KEY[gather_name]) if c.act is not None else None
    if tp == 1 or peer is None or not cfg.gather_in_place:
        return None
    rows = peer.shape[0] // tp
    return _use(peer, c.stream)[cfg.tp_rank * rows:(cfg.tp_rank + 1) * rows]


def _h_norm(c):
    p = "attn" if c.op == 1 else "mlp"
    fn = c.dcfunc.ln_attn if c.op == 1 else c.dcfunc.ln_mlp
    act = c.act
    output, act[f"{p}_mu"], act[f"{p}_rsigma"], act[f"ln_{p}_input"], act[f"ln_{p}_residual"], _ = fn(
        c.config, (c.x, c.weight[f"ln_{p}_weight"], c.weight.get(f"ln_{p}_bias")), c.stream,
        out=_gather_slot(c, f"allgather_{p}"))
    return output


def _h_gemm_attn_c(c):
    c.act["gemm_attn_c_input"] = c.x
    return c.dcfunc.gemm_attn_column(c.config, (c.x, c.weight["column_attn_weight"]), c.stream)


def _h_rope(c):
    return c.dcfunc.rope(c.config, (c.x,), c.stream)


def _h_attn(c):
    act = c.act
    (output, act["q_padded"], act["k_padded"], act["v_padded"], act["out_padded"], act["rng_state"],
     act["softmax_lse"]) = c.dcfunc.attn(c.config, (c.x, c.weight["cu_seqlens_q"], c.weight["cu_seqlens_kv"]), c.stream,
                                         apply_rope=c.config.groups_per_rank != 1)
    return output


def _h_gemm_attn_l(c):
    output, c.act["linear_attn_input"] = c.dcfunc.gemm_attn_linear(c.config, (c.x, c.weight["linear_attn_weight"]), c.stream)
    return output


def _h_gemm_mlp_c(c):
    c.act["gemm_mlp_c_input"] = c.x
    return c.dcfunc.gemm_mlp_column(c.config, (c.x, c.weight["column_mlp_weight"]), c.stream)


def _h_gemm_mlp_l(c):
    output, c.act["linear_mlp_input"] = c.dcfunc.gemm_mlp_linear(c.config, (c.x, c.weight["linear_mlp_weight"]), c.stream)
    return output


def _h_bda_mlp(c):
    output, c.act["mlp_mask"] = c.dcfunc.bda_mlp(c.config, (c.x, c.g("ln_mlp_residual")), c.stream)
    return output


def _h_bda_attn(c):
    output, c.act["attn_mask"] = c.dcfunc.bda_attn(c.config, (c.x, c.g("ln_attn_residual")), c.stream)
    return output


def _h_reduce_scatter(c):
    return c.dcfunc.reduce_scatter(c.config, (c.x,), c.stream, bwd_strand=bool(c.name) and c.name.endswith("_bwd"))


def _h_all_gather(c):
    peer = c.act.get(_PEER_KEY.get(c.name, ""))
    return c.dcfunc.allgather(c.config, (c.x, _use(peer, c.stream)), c.stream,
                              bwd_strand=bool(c.name) and c.name.endswith("_bwd"))


def _h_swiglu(c):
    output = c.dcfunc.swiglu(c.config, (c.x,), c.stream)
    c.act["swiglu_input"] = c.x
    return output


_DGRAD_WEIGHT = {13: "column_mlp_weight", 15: "linear_mlp_weight", 17: "column_attn_weight", 19: "linear_attn_weight"}


def _h_dgrad(c):
    return c.dcfunc._dgrad(c.config, (c.x, c.weight[_DGRAD_WEIGHT[c.op]]), c.stream)


def _run_or_park(c, fn, args):
    """A weight gradient runs now, or -- when the plan names its placeholder -- is parked until the placeholder
    op (or the end of the block list) runs it (dstb.py:543-598)."""
    if _WGRAD_PLACEHOLDER[c.op] in c.movable:
        c.act.setdefault("_parked", {})[_WGRAD_PLACEHOLDER[c.op]] = (fn, (c.config, args, c.stream))
    else:
        fn(c.config, args, c.stream)
    return None


def _h_wgrad_column(c):
    # (saved GEMM input, incoming gradient, main_grad)
    if c.op == 14:
        args = (c.g("gemm_mlp_c_input"), c.g("swiglu_dgrad"), c.weight["column_mlp_weight"].main_grad)
        return _run_or_park(c, c.dcfunc.gemm_wgrad_mlp_c, args)
    c.act.pop("attn_dgrad", None)          # kept by the last ring call for this weight gradient
    args = (c.g("gemm_attn_c_input"), c.x, c.weight["column_attn_weight"].main_grad)
    return _run_or_park(c, c.dcfunc.gemm_wgrad_attn_c, args)


def _h_wgrad_linear(c):
    key, wkey = ("linear_mlp_input", "linear_mlp_weight") if c.op == 16 else ("linear_attn_input", "linear_attn_weight")
    args = (c.x, c.g(key), c.weight[wkey].main_grad)
    return _run_or_park(c, c.dcfunc.gemm_wgrad_mlp_l if c.op == 16 else c.dcfunc.gemm_wgrad_attn_l, args)


def _h_placeholder(c):
    parked = c.act.get("_parked", {}).pop(_PLACEHOLDER_ID[c.op], None)
    if parked is not None:
        fn, (cfg, args, _) = parked
        fn(cfg, args, c.stream)
    return None


def _h_swiglu_bwd(c):
    output = c.dcfunc.swiglu_bwd(c.config, (c.g("swiglu_input"), c.x), c.stream)
    c.act["swiglu_dgrad"] = output
    return output


def _h_bda_mlp_bwd(c):
    output, c.act["mlp_residual_bwd"] = c.dcfunc.bda_mlp_bwd(c.config, (c.x, c.act.get("mlp_mask")), c.stream)
    return output


def _h_bda_attn_bwd(c):
    output, c.act["attn_residual_bwd"] = c.dcfunc.bda_attn_bwd(c.config, (c.x, c.act.get("attn_mask")), c.stream)
    return output


def _h_attn_bwd(c):
    return c.dcfunc.attn_bwd(c.config, (c.x, c.g("q_padded"), c.g("k_padded"), c.g("v_padded"), c.g("out_padded"),
                                        c.g("softmax_lse"), c.weight["cu_seqlens_q"], c.weight["cu_seqlens_kv"],
                                        c.act.get("rng_state")), c.stream, apply_rope=c.config.groups_per_rank != 1)


def _h_rope_bwd(c):
    return c.dcfunc.rope_bwd(c.config, (c.x,), c.stream)


def _h_ring_fwd(c):
    act, x = c.act, c.x
    last = (0 if isinstance(x, torch.Tensor) else x[7]) == c.config.context_parallel_size - 1
    visiting = act.get("cp_kv_chunks")
    for t in visiting or ():
        _use(t, c.stream)
    output = c.dcfunc.ring_attn_fwd(c.config, (x, c.weight["cu_seqlens_q"], c.weight["cu_seqlens_kv"],
                                               c.weight.get("rope_positions"), visiting), c.stream)
    if last:       # dstb.py:471-481
        output, act["q"], act["kv"], act["softmax_lse"], act["rng_states"] = output
        act["out"] = output
    return output


def _h_ring_bwd(c):
    act, x = c.act, c.x
    last = (0 if isinstance(x, torch.Tensor) else x[4]) == c.config.context_parallel_size
    for t in act["kv"]:
        _use(t, c.stream)
    output = c.dcfunc.ring_attn_bwd(c.config, (x, c.g("out"), c.g("q"), act["kv"], c.g("softmax_lse"), act.get("rng_states"),
                                               c.weight["cu_seqlens_q"], c.weight["cu_seqlens_kv"],
                                               c.weight.get("rope_positions")), c.stream)
    if last:       # dstb.py:492-504
        for key in ("out", "q", "kv", "softmax_lse", "rng_states"):
            act.pop(key, None)
        act["attn_dgrad"] = output
    return output


def _h_norm_bwd(c):
    p = "mlp" if c.op == 25 else "attn"
    lw, lb = c.weight[f"ln_{p}_weight"], c.weight.get(f"ln_{p}_bias")
    mu = c.act.get(f"{p}_mu")
    data = (c.x, c.g(f"ln_{p}_input"), _use(mu, c.stream), c.g(f"{p}_rsigma"), lw, lb, c.g(f"{p}_residual_bwd"),
            lw.main_grad, lb.main_grad if lb is not None else None)
    if c.op == 25:       # its result is what allgather_attn_bwd gathers (bda_attn_bwd in between passes it through)
        return c.dcfunc.ln_mlp_bwd(c.config, data, c.stream, out=_gather_slot(c, "allgather_attn_bwd"))
    return c.dcfunc.ln_attn_bwd(c.config, data, c.stream)


def _h_bda_attn_ln_mlp(c):
    """bda_attn followed by ln_mlp in one column of a plan: what the two handlers would save, from one kernel."""
    act = c.act
    output, act["mlp_mu"], act["mlp_rsigma"], act["ln_mlp_input"], act["ln_mlp_residual"] = c.dcfunc.bda_attn_ln_mlp(
        c.config, (c.x, c.g("ln_attn_residual"), c.weight["ln_mlp_weight"], c.weight.get("ln_mlp_bias")), c.stream,
        out=_gather_slot(c, "allgather_mlp"))
    act["attn_mask"] = None
    act.pop("ln_attn_residual", None)
    return output


# (name, name of the op that follows it in the same column) -> handler that runs both
_FUSED = {("bda_attn", "ln_mlp"): _h_bda_attn_ln_mlp}


# op id -> handler (the reference: one ``if operation == N`` after another, dstb.py:431-657)
_HANDLERS = {
    1: _h_norm, 2: _h_norm, 3: _h_gemm_attn_c, 4: _h_gemm_attn_l, 5: _h_gemm_mlp_c, 6: _h_gemm_mlp_l, 7: _h_attn,
    8: _h_bda_mlp, 9: _h_bda_attn, 10: _h_reduce_scatter, 11: _h_all_gather, 12: _h_swiglu,
    13: _h_dgrad, 15: _h_dgrad, 17: _h_dgrad, 19: _h_dgrad,
    14: _h_wgrad_column, 18: _h_wgrad_column, 16: _h_wgrad_linear, 20: _h_wgrad_linear,
    114: _h_placeholder, 116: _h_placeholder, 118: _h_placeholder, 120: _h_placeholder,
    21: _h_swiglu_bwd, 22: _h_bda_mlp_bwd, 23: _h_bda_attn_bwd, 24: _h_attn_bwd, 25: _h_norm_bwd, 26: _h_norm_bwd,
    29: _h_ring_fwd, 30: _h_ring_bwd, 31: _h_rope, 32: _h_rope_bwd,
}


class DCoperation:
    """Dispatch one op id: fetch its inputs (previous op's output, weights, saved
    activations), run the adapter, save / free activations (dstb.py:427-660)."""

    @staticmethod
    def perform_fused(dcfunc, names, config, weight, activation_dict, **kwargs):
        """Two ops that a plan lists next to each other in one column, run as one kernel (the plan keeps both
        names; the result is what running them one after the other gives, bit for bit)."""
        handler = _FUSED[tuple(names)]
        return handler(_Ctx(dcfunc, None, config, weight, activation_dict, kwargs.get("output"), kwargs["stream"],
                            names[0], kwargs.get("movable", ())))

    @staticmethod
    def perform_operation(dcfunc, operation, config, weight, activation_dict, **kwargs):
        op = operation.value if isinstance(operation, FuncChoice) else int(operation)
        handler = _HANDLERS.get(op)
        if handler is None:
            raise ValueError(f"operation {op} is not part of the single-GPU decoder-layer path")
        output = handler(_Ctx(dcfunc, op, config, weight, activation_dict, kwargs.get("output"), kwargs["stream"],
                              kwargs.get("name"), kwargs.get("movable", ())))
        for key in _FREE_AFTER.get(op, ()):
            activation_dict.pop(key, None)
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
    skip = False
    for idx, now_op in enumerate(col):
        if skip:                    # ran together with the op before it
            skip = False
            continue
        src = now_op.get_output()
        inp = first_input if src is None else src
        st = stream_of(now_op)
        nxt_in_col = col[idx + 1] if idx + 1 < len(col) else None
        if (nxt_in_col is not None and (now_op.name, nxt_in_col.name) in _FUSED and getattr(config, "fuse_adjacent", True)
                and hasattr(dcoperation, "perform_fused") and nxt_in_col in now_op.get_next_op()):
            output = dcoperation.perform_fused(DCFunc, (now_op.name, nxt_in_col.name), config, weight, act, output=inp,
                                               stream=st, movable=movable)
            now_op.set_output(None)
            now_op = nxt_in_col         # successors and result bookkeeping are those of the second op
            skip = True
            handle = None
            now_op.set_output(None)
            nxt = now_op.get_next_op()
            if output is not None and len(nxt) == 0:
                result[0] = output
            for nop in nxt:
                nop.set_output(output)
                nop.set_handle(handle)
            continue
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


class DSTB_(torch.autograd.Function):
    """One module of the folded model (dstb.py:1294-1366).  The model is walked twice per micro-batch: the
    forward traversal calls ``forward`` (the module's FIRST layer takes the new micro-batch forward, its SECOND
    layer takes the previous micro-batch backward), the autograd traversal that follows calls ``backward`` with
    the two weight sets exchanged.  Inputs and results travel through ``GLOBAL_VARIABLES['inputs']`` =
    [backward strand's gradient, forward strand's hidden states]; activation dicts are pushed on the stack of
    the micro-batch that made them and popped by the traversal that differentiates them."""

    @staticmethod
    def _walk(config, fwd_weight, bwd_weight, plan, stream1, stream2, push_to, pop_from):
        bwd_input, fwd_input = GLOBAL_VARIABLES['inputs']
        new_act = {}
        if bwd_input is None:                               # only the new micro-batch: forward
            fwd_result, _ = exec(config, DCoperation, fwd_weight, None, fwd_input, None, plan.fwd_only, stream1,
                                 stream2, None, new_act, movable=plan.movable)
            GLOBAL_VARIABLES[push_to][-1].push(new_act)
            GLOBAL_VARIABLES['inputs'] = [None, fwd_result]
            return
        act = GLOBAL_VARIABLES[pop_from][0].pop()           # activations of the previous micro-batch
        if GLOBAL_VARIABLES[pop_from][0].is_empty():
            GLOBAL_VARIABLES[pop_from].pop(0)
        if fwd_input is None:                               # only the previous micro-batch: backward
            _, bwd_result = exec(config, DCoperation, None, bwd_weight, None, bwd_input, plan.bwd_only, stream1,
                                 stream2, act, None, movable=plan.movable)
            GLOBAL_VARIABLES['inputs'] = [bwd_result, None]
            return
        fwd_result, bwd_result = exec(config, DCoperation, fwd_weight, bwd_weight, fwd_input, bwd_input,
                                      plan.dcblocks, stream1, stream2, act, new_act, movable=plan.movable)
        GLOBAL_VARIABLES[push_to][-1].push(new_act)
        GLOBAL_VARIABLES['inputs'] = [bwd_result, fwd_result]

    @staticmethod
    def forward(ctx, placeholder, config, bwd_weight, fwd_weight, plan, stream1, stream2):
        ctx.args = (config, fwd_weight, bwd_weight, plan, stream1, stream2)
        with torch.no_grad():
            DSTB_._walk(config, fwd_weight, bwd_weight, plan, stream1, stream2, 'fwd_activations', 'bwd_activations')
        return placeholder.view_as(placeholder)

    @staticmethod
    def backward(ctx, *grads):
        config, fwd_weight, bwd_weight, plan, stream1, stream2 = ctx.args
        with torch.no_grad():                               # the two weight sets change places (dstb.py:1333-1335)
            DSTB_._walk(config, bwd_weight, fwd_weight, plan, stream1, stream2, 'bwd_activations', 'fwd_activations')
        return grads[0], None, None, None, None, None, None


_DSTB_WEIGHTS = ("ln_attn_weight", "column_attn_weight", "linear_attn_weight", "ln_mlp_weight", "column_mlp_weight",
                 "linear_mlp_weight")


class DSTB(torch.nn.Module):
    """Two decoder layers in one module (dstb.py:1368-1468): ``*_first`` is the layer the forward traversal runs,
    ``*_second`` the one the autograd traversal runs, so a model of n such modules is the 2n-layer network
    first_0 .. first_{n-1}, second_{n-1} .. second_0.  Parameters are ``torch.nn.Parameter`` with a ``main_grad``
    buffer each (Megatron's distributed optimizer provides it in the reference)."""

    def __init__(self, config: LayerConfig, stream1, stream2, plan=None, seed: int = 0, device="cuda"):
        super().__init__()
        from .layer import make_weights
        self.config, self.stream1, self.stream2 = config, stream1, stream2
        self.weight_first, self.weight_second = {}, {}
        for tag, wd, sd in (("first", self.weight_first, seed), ("second", self.weight_second, seed + 1)):
            w = make_weights(config, sd, device)
            names = _DSTB_WEIGHTS + (("ln_attn_bias", "ln_mlp_bias") if config.layernorm_bias else ())
            for k in names:
                p = torch.nn.Parameter(w[k])
                p.main_grad = torch.zeros_like(w[k])
                if config.resident_weight_transposes and k in _DGRAD_WEIGHT.values():
                    keep_transposed(p)
                if k.startswith("ln_"):
                    p.sequence_parallel = config.tensor_model_parallel_size > 1
                setattr(self, f"{k}_{tag}", p)
                wd[k] = p
            for k in ("cu_seqlens_q", "cu_seqlens_kv", "rope_positions"):
                if k in w:
                    wd[k] = w[k]
        self.plan = init_DCBlocks(plan, stream1, stream2, config.context_parallel_size)
        self.dcblocks, self.fwd_only_dcblocks, self.bwd_only_dcblocks = self.plan

    def forward(self, inputs):
        return DSTB_.apply(inputs, self.config, self.weight_second, self.weight_first, self.plan, self.stream1,
                           self.stream2)
