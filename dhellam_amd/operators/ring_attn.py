"""Ring / context-parallel attention block step, forward and backward, on one GPU.

Mirrors dhellam/operators/ring_attn.py:43-201 (``fa_cp_block_fwd``) and :204-411
(``fa_cp_block_bwd``): the same step-wise state machine over ``i``, the same three
zig-zag cases, the same argument order and carry lists.  Differences, all forced by
"one GPU, no collectives":

* ``cp_group`` is a :class:`RingGroup` (rank, size) instead of a process group, and
  nothing is sent: ``p2p_comm_buffers[i]`` must already hold the KV chunk that visits
  at forward step ``i`` (the one that originated on rank ``(rank - i) % size``), shape
  ``[2, b, 2, sk/2, hk, d]`` (non-causal: ``[2, b, sk, hk, d]``).  The returned
  ``p2p_reqs`` is an empty list.
* K/V may have fewer heads than Q (GQA); the reference views KV with Q's head count
  (ring_attn.py:95).
* softmax scale and dropout are parameters (``softmax_scale`` default 1/sqrt(d); dropout
  is not implemented) instead of the hard-coded 0.125 / 0.1 (ring_attn.py:100).
* The merge of the partial outputs runs once, fused, in fp32 on the last step, instead of one
  pass over ``out`` per step (ring_attn.py:171-195).  The carried ``softmax_lse`` /
  ``softmax_lse_`` are kept up to date as in the reference (step i folds step i - 1's
  log-sum-exp into them, ring_attn.py:146-164), in fp32 instead of fp64, so a caller that
  looks at the carry between steps sees the running value; the value returned after the
  last step is the one the fused merge computes from all steps.
* Backward keeps one dKV buffer per visiting chunk (``dkv_`` is a list) instead of adding
  into a buffer that travels round the ring (ring_attn.py:239-272).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from .. import _Clib


@dataclass(frozen=True)
class RingGroup:
    """Stand-in for the context-parallel process group: this rank's place in the ring."""
    rank: int
    size: int


def get_distributed_rank(group: RingGroup) -> int:
    return group.rank


def get_distributed_world_size(group: RingGroup) -> int:
    return group.size


def _rows(x):
    """[b, n, h, d] (possibly a strided view) -> [b*n, h, d] without a copy when b == 1."""
    b, n, h, d = x.shape
    if b == 1:
        return x[0]
    return x.contiguous().view(b * n, h, d)


def _scale(q, softmax_scale):
    return float(softmax_scale) if softmax_scale is not None else 1.0 / math.sqrt(q.shape[-1])


def fa_cp_block_fwd(q, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, p2p_comm_buffers, out_per_step,
                    softmax_lse_per_step, rng_states, softmax_lse, softmax_lse_, i, causal, cp_group,
                    cp_global_ranks, stream, softmax_scale=None):
    """One forward step.  q [b, 2, sq/2, hq, d] (causal) or [b, sq, hq, d].

    Returns ``([q, p2p_comm_buffers, out_per_step, softmax_lse_per_step, rng_states,
    softmax_lse, softmax_lse_, i + 1], p2p_reqs)`` for i < size - 1 and
    ``(out, q, kv, softmax_lse, rng_states)`` on the last step, as the reference does
    (ring_attn.py:199-201)."""
    assert q.shape[-1] % 8 == 0, "hidden size per attention head should be multiple of 8"
    rank = get_distributed_rank(cp_group)
    cp_size = get_distributed_world_size(cp_group)
    scale = _scale(q, softmax_scale)
    kv_inputs = p2p_comm_buffers[i]
    if i == 0:
        out_per_step = [None] * cp_size
        softmax_lse_per_step = [None] * cp_size
        rng_states = [None] * cp_size
    if stream is None:
        stream = torch.cuda.current_stream()
    hq, d = q.shape[-2], q.shape[-1]

    with torch.cuda.stream(stream):
        if causal:
            b, _, c = q.shape[0], q.shape[1], q.shape[2]
            if i == 0:       # diagonal: all q rows x all kv rows, causal
                q_in = _rows(q.view(b, 2 * c, hq, d))
                k_in = _rows(kv_inputs[0].reshape(b, -1, *kv_inputs.shape[-2:]))
                v_in = _rows(kv_inputs[1].reshape(b, -1, *kv_inputs.shape[-2:]))
                cq, ck, mq, mk, cz = cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, True
            elif i <= rank:  # lower: all q rows x first half of kv, no mask
                q_in = _rows(q.view(b, 2 * c, hq, d))
                k_in = _rows(kv_inputs[0][:, 0])
                v_in = _rows(kv_inputs[1][:, 0])
                cq, ck, mq, mk, cz = cu_seqlens_q, cu_seqlens_k // 2, max_seqlen_q, max_seqlen_k // 2, False
            else:            # upper: second half of q x all kv rows, no mask
                q_in = _rows(q[:, 1])
                k_in = _rows(kv_inputs[0].reshape(b, -1, *kv_inputs.shape[-2:]))
                v_in = _rows(kv_inputs[1].reshape(b, -1, *kv_inputs.shape[-2:]))
                cq, ck, mq, mk, cz = cu_seqlens_q // 2, cu_seqlens_k, max_seqlen_q // 2, max_seqlen_k, False
        else:
            b = q.shape[0]
            q_in = _rows(q)
            k_in, v_in = _rows(kv_inputs[0]), _rows(kv_inputs[1])
            cq, ck, mq, mk, cz = cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, False
        res = _Clib.pymha_varlen_fwd(q_in, k_in, v_in, cq, ck, mq, mk, 0.0, scale, cz, False, 0, False)
        out_per_step[i], softmax_lse_per_step[i], rng_states[i] = res[0], res[5], res[7]

        # running log-sum-exp over the steps before this one (ring_attn.py:146-164): step i folds step i - 1
        if i == 1:
            softmax_lse = softmax_lse_per_step[0].clone()
            if causal:
                softmax_lse_ = softmax_lse.view(*softmax_lse.shape[:-1], 2, -1)
        elif i > 1:
            prev = softmax_lse_per_step[i - 1]
            if causal and i - 1 > rank:            # a half-q step: only the second half of the rows
                torch.logaddexp(softmax_lse_[..., 1, :], prev, out=softmax_lse_[..., 1, :])
            else:
                torch.logaddexp(softmax_lse, prev, out=softmax_lse)

        if i == cp_size - 1:
            sq = max_seqlen_q
            row_begin, rows = [], []
            for s in range(cp_size):
                half = causal and s > rank
                row_begin.append(sq // 2 if half else 0)
                rows.append(sq // 2 if half else sq)
            out = torch.empty((b * sq, hq, d), dtype=q.dtype, device=q.device)
            softmax_lse = torch.empty((b, hq, sq), dtype=torch.float32, device=q.device)
            _Clib.pyattn_merge(out_per_step, softmax_lse_per_step, row_begin, rows, out, softmax_lse)
            kv = p2p_comm_buffers[-1]
            return out, q, kv, softmax_lse, rng_states
    return [q, p2p_comm_buffers, out_per_step, softmax_lse_per_step, rng_states, softmax_lse, softmax_lse_,
            i + 1], []


def fa_cp_block_bwd(dout, out, q, dq, kv, dkv_, softmax_lse, rng_states, cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
                    max_seqlen_k, p2p_comm_buffers, i, causal, cp_group, cp_global_ranks, stream,
                    softmax_scale=None):
    """One backward call, i in [0, size].  Call i < size runs the backward of forward step
    ``size - 1 - i`` (ring_attn.py:303,323,343) with the MERGED ``out`` / ``softmax_lse``
    and accumulates into ``dq``; the last call (i == size) only returns ``(dq, dkv)``.

    ``p2p_comm_buffers`` is the forward list (indexed by forward step).  ``dkv_`` is None
    on the first call, afterwards the list of per-chunk gradients ``[2, b, 2, sk/2, hk, d]``
    (entry s filled once forward step s has been differentiated; an 'L' step leaves the
    second half zero).  ``dq`` may be None on the first call (it is allocated, like q).
    Returns ``([dout, dq, dkv_, p2p_comm_buffers, i + 1], [])`` or ``(dq, dkv_)``."""
    rank = get_distributed_rank(cp_group)
    cp_size = get_distributed_world_size(cp_group)
    if i == cp_size:
        if causal:
            dq = dq.view(q.shape[0], -1, *q.shape[-2:])
        return dq, dkv_
    scale = _scale(q, softmax_scale)
    if stream is None:
        stream = torch.cuda.current_stream()
    hq, d = q.shape[-2], q.shape[-1]
    step = cp_size - 1 - i
    kv_in = p2p_comm_buffers[step]
    sp = stream.cuda_stream

    with torch.cuda.stream(stream):
        if dkv_ is None:
            dkv_ = [None] * cp_size
        if dq is None:
            dq = torch.empty_like(q)
        out = out.view(*q.shape)
        dout = dout.view(*q.shape)
        dkv = torch.empty_like(kv_in)
        if causal:
            b, c = q.shape[0], q.shape[2]
            hk = kv_in.shape[-2]
            if step == 0:
                case = "D"
            elif step <= rank:
                case = "L"
            else:
                case = "U"
            if case == "U":
                q_, o_, do_ = _rows(q[:, 1]), _rows(out[:, 1]), _rows(dout[:, 1])
                lse_ = softmax_lse.view(b, hq, 2, c)[:, :, 1].contiguous()
                cq, mq = cu_seqlens_q // 2, max_seqlen_q // 2
            else:
                q_, o_, do_ = (_rows(x.view(b, 2 * c, hq, d)) for x in (q, out, dout))
                lse_ = softmax_lse
                cq, mq = cu_seqlens_q, max_seqlen_q
            if case == "L":
                k_, v_ = _rows(kv_in[0][:, 0]), _rows(kv_in[1][:, 0])
                dk_, dv_ = _rows(dkv[0][:, 0]), _rows(dkv[1][:, 0])
                dkv[:, :, 1].zero_()
                ck, mk = cu_seqlens_k // 2, max_seqlen_k // 2
            else:
                k_, v_ = (_rows(x.reshape(b, 2 * c, hk, d)) for x in (kv_in[0], kv_in[1]))
                dk_, dv_ = (_rows(x.view(b, 2 * c, hk, d)) for x in (dkv[0], dkv[1]))
                ck, mk = cu_seqlens_k, max_seqlen_k
            cz = case == "D"
            first_touch_all = i == 0 and case != "U"   # this step writes every dq row first
            if case == "U":
                dq_rows = dq[:, 1]
            else:
                dq_rows = dq.view(b, 2 * c, hq, d)
        else:
            b = q.shape[0]
            q_, o_, do_ = _rows(q), _rows(out), _rows(dout)
            lse_ = softmax_lse
            k_, v_ = _rows(kv_in[0]), _rows(kv_in[1])
            dk_, dv_ = _rows(dkv[0]), _rows(dkv[1])
            cq, mq, ck, mk, cz = cu_seqlens_q, max_seqlen_q, cu_seqlens_k, max_seqlen_k, False
            first_touch_all = i == 0
            dq_rows = dq
        # With batch > 1 the first-half views of an 'L' step are not contiguous: _rows() then hands out
        # packed temporaries, and the results are copied back into the views.
        dkv_is_temp = dk_.data_ptr() != dkv[0].data_ptr()
        # dq: the first contribution to a row is a store, later ones add (ring_attn.py:391-408), both inside the
        # kernel when the rows form one packed run (always for batch 1): no temporary and no extra pass over dq.
        first_store = first_touch_all or (causal and i == 0)
        if causal and i == 0 and not first_touch_all:      # first call is a 'U' step: only the second half exists yet
            dq[:, 0].zero_()
        if dq_rows.is_contiguous() or dq_rows.shape[0] == 1:
            tgt = dq_rows.reshape(-1, hq, d) if dq_rows.is_contiguous() else dq_rows[0]
            _Clib._attn_bwd_raw(do_, q_, k_, v_, o_, lse_, tgt, dk_, dv_, None, cq, ck, mq, mk, scale, cz, sp,
                                accumulate_dq=not first_store)
        else:
            dq_step = torch.empty(q_.shape, dtype=q.dtype, device=q.device)
            _Clib._attn_bwd_raw(do_, q_, k_, v_, o_, lse_, dq_step, dk_, dv_, None, cq, ck, mq, mk, scale, cz, sp)
            dq_step = dq_step.view(dq_rows.shape)
            if first_store:
                dq_rows.copy_(dq_step)
            else:
                dq_rows.add_(dq_step)
        if dkv_is_temp:
            assert causal and case == "L"
            dkv[0][:, 0].copy_(dk_.view(b, c, hk, d))
            dkv[1][:, 0].copy_(dv_.view(b, c, hk, d))
        dkv_[step] = dkv
    return [dout, dq, dkv_, p2p_comm_buffers, i + 1], []
