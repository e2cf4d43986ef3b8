"""Vocab-parallel cross entropy and the masked mean loss: dhellam/operators/loss.py:15-164.

Same calling convention as the reference (dict in, dict out, ``bwd(context, dout)``).  The
reference materialises the softmax in the forward and turns it into the gradient in the
backward; with ``keep_softmax=False`` the forward keeps only two numbers per row (maximum and
exponential sum) and the backward recomputes the softmax from the logits, which removes one
[rows, vocab] write and one read from the pair and leaves nothing of that size alive in
between.  ``output_dict["softmax"]`` is then None.

The all-reduces over the tensor-parallel group (loss.py:22-24,52-56,61-66) are the caller's:
with a world size above one the outputs are this rank's share.  The ranks join their row
statistics as

    M = max_r row_max_r,   S = sum_r sum_exp_r * exp(row_max_r - M),
    P = sum over the rank that holds the target of (predicted_r + row_max_r - M),
    loss = log S - P,

(two all-reduces of [rows] floats instead of the reference's three) and each rank's share of
the gradient comes from ``cross_entropy_bwd`` with ``row_max`` / ``sum_exp`` in its context
replaced by M / S (``keep_softmax=False``; a kept softmax is normalised by the rank's own sum).
"""
from __future__ import annotations

import torch

from .. import _lib
from ..common.parallel_state import get_tensor_model_parallel_rank, get_tensor_model_parallel_world_size
from .embedding import vocab_range_from_per_partition_vocab_size


def cross_entropy_fwd(inputs, label_smoothing=0.0, keep_softmax=True):
    logits, target = inputs["vocab_parallel_logits"], inputs["target"]
    _lib.need_cuda(logits, target)
    assert logits.stride(-1) == 1 and target.dtype == torch.int64 and target.shape == logits.shape[:-1]
    cols = logits.shape[-1]
    x = logits.reshape(-1, cols)                       # a view for contiguous logits
    if x.stride(-1) != 1:
        x = x.contiguous()
    tgt = target.contiguous()
    rows = x.shape[0]
    start, _ = vocab_range_from_per_partition_vocab_size(cols, get_tensor_model_parallel_rank(),
                                                        get_tensor_model_parallel_world_size())
    dev = logits.device
    stats = torch.empty((4, max(rows, 1)), dtype=torch.float32, device=dev)   # loss, row_max, sum_exp, predicted
    softmax = torch.empty((rows, cols), dtype=logits.dtype, device=dev) if keep_softmax else None
    mask = torch.empty(rows, dtype=torch.bool, device=dev)
    masked_target = torch.empty(rows, dtype=torch.int64, device=dev)
    _lib.check(_lib.load().dh_cross_entropy_fwd(
        x.data_ptr(), tgt.data_ptr(), rows, cols, x.stride(0), start, float(label_smoothing), _lib.dt(x),
        stats[0].data_ptr(), stats[1].data_ptr(), stats[2].data_ptr(), stats[3].data_ptr(),
        softmax.data_ptr() if keep_softmax else None, cols, mask.data_ptr(), masked_target.data_ptr(),
        torch.cuda.current_stream().cuda_stream))
    return {
        "loss": stats[0, :rows].view(target.shape),
        "label_smoothing": label_smoothing,
        "vocab_size": cols,
        "softmax": softmax.view(logits.shape) if keep_softmax else None,
        "target_mask": mask.view(target.shape),
        "masked_target_1d": masked_target,
        "row_max": stats[1, :rows], "sum_exp": stats[2, :rows], "predicted": stats[3, :rows].view(target.shape),
    }


def cross_entropy_bwd(context, dout, grad_out=None):
    """Returns d loss / d logits scaled by ``dout`` per row.  With the softmax kept it is written
    over the softmax, as in the reference (loss.py:105-126); otherwise into ``grad_out`` (default:
    a new tensor; pass the logits themselves to overwrite them)."""
    inputs, out = context[0], context[1]
    logits, target = inputs["vocab_parallel_logits"], inputs["target"]
    cols = out["vocab_size"]
    start, _ = vocab_range_from_per_partition_vocab_size(cols, get_tensor_model_parallel_rank(),
                                                        get_tensor_model_parallel_world_size())
    d = dout.to(torch.float32).contiguous()
    tgt = target.contiguous()
    rows = tgt.numel()
    assert d.numel() == rows
    lib, st = _lib.load(), torch.cuda.current_stream().cuda_stream
    if out["softmax"] is not None:
        sm = out["softmax"]
        s2 = sm.view(-1, cols)
        _lib.check(lib.dh_cross_entropy_bwd(s2.data_ptr(), s2.stride(0), 0, None, None, tgt.data_ptr(), d.data_ptr(),
                                            rows, cols, start, float(out["label_smoothing"]), _lib.dt(sm),
                                            s2.data_ptr(), s2.stride(0), st))
        return sm
    x = logits.reshape(-1, cols)
    if x.stride(-1) != 1:
        x = x.contiguous()
    g = torch.empty((rows, cols), dtype=logits.dtype, device=logits.device) if grad_out is None else grad_out.view(-1, cols)
    assert g.dtype == x.dtype and g.stride(-1) == 1
    _lib.check(lib.dh_cross_entropy_bwd(x.data_ptr(), x.stride(0), 1, out["row_max"].data_ptr(), out["sum_exp"].data_ptr(),
                                        tgt.data_ptr(), d.data_ptr(), rows, cols, start, float(out["label_smoothing"]),
                                        _lib.dt(x), g.data_ptr(), g.stride(0), st))
    return g.view(logits.shape)


def mask_scale_loss_fwd(inputs):
    """loss = sum(losses * mask) / sum(mask) / num_microbatch * loss_scale (loss.py:131-153).  The NaN
    assertion of the reference needs a host sync and is left to the caller."""
    loss_mask, losses = inputs["loss_mask"], inputs["output_tensor"]
    _lib.need_cuda(loss_mask, losses)
    x = losses.to(torch.float32).contiguous().view(-1)
    m = loss_mask.reshape(-1).to(torch.float32).contiguous()
    assert x.numel() == m.numel() and x.numel() > 0
    scale = float(inputs["loss_scale"]) / float(inputs["num_microbatch"])
    out = torch.empty(2, dtype=torch.float32, device=x.device)
    _lib.check(_lib.load().dh_masked_mean_fwd(x.data_ptr(), m.data_ptr(), x.numel(), scale, out.data_ptr(),
                                              torch.cuda.current_stream().cuda_stream))
    return {"loss": out[0], "mask_sum": out[1:2], "mask_f32": m}


def mask_scale_loss_bwd(context, dout=None):
    """d loss / d output_tensor; like the reference (loss.py:155-164) the incoming gradient is one."""
    inputs, out = context[0], context[1]
    losses, m = inputs["output_tensor"], out["mask_f32"]
    scale = float(inputs["loss_scale"]) / float(inputs["num_microbatch"])
    g = torch.empty(m.numel(), dtype=torch.float32, device=m.device)
    _lib.check(_lib.load().dh_masked_mean_bwd(m.data_ptr(), out["mask_sum"].data_ptr(), m.numel(), scale, g.data_ptr(),
                                              torch.cuda.current_stream().cuda_stream))
    return g.view(losses.shape).to(losses.dtype)
