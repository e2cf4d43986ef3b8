"""Oracle for the head block: vocab-parallel word embedding, vocab-parallel cross entropy,
masked mean loss (dhellam/operators/embedding.py, dhellam/operators/loss.py,
dhellam/core/dshb.py:98-112).

Test infrastructure: eager PyTorch on the CPU, fp64 unless stated.  The reference runs one
process per tensor-parallel rank and joins them with all-reduces; here the ranks are the
entries of a list and a collective is an explicit reduction over that list, so the
sharded algorithm is restated whole and can be pinned against the unsharded definition.
With ``collectives=False`` every all-reduce is the identity: that is what ONE rank
computes before it hears from the others, the share a single GPU can show.
"""
from __future__ import annotations

import torch

F64 = torch.float64


def vocab_range(per_partition_vocab_size: int, rank: int):
    """loss.py:8-13 / embedding.py:8-13."""
    first = rank * per_partition_vocab_size
    return first, first + per_partition_vocab_size


# --------------------------------------------------------------------------------------
# word embedding.  embedding.py:16-39 (forward), :42-49 (backward through autograd)
# --------------------------------------------------------------------------------------
def word_embedding_fwd(vocab, token_ids, tp_rank=0, tp_world=1, dtype=F64):
    """vocab: this rank's [rows, hidden] slice.  Ids outside the slice give zero rows
    (the all-reduce over ranks, outside this operator, fills them in)."""
    first, last = vocab_range(vocab.shape[0], tp_rank)
    if tp_world > 1:
        outside = (token_ids < first) | (token_ids >= last)
        local = token_ids.clone() - first
        local[outside] = 0
    else:
        local = token_ids
    out = vocab.to(dtype)[local]
    if tp_world > 1:
        out[outside, :] = 0.0
    return out


def word_embedding_bwd(dout, token_ids, vocab_rows, tp_rank=0, tp_world=1, dtype=F64):
    """Gradient of the slice: row v receives the sum of dout over the positions whose id is
    first + v (what autograd's index backward computes in embedding.py:48)."""
    first, last = vocab_range(vocab_rows, tp_rank)
    ids = token_ids.reshape(-1)
    d = dout.to(dtype).reshape(ids.numel(), dout.shape[-1])
    g = torch.zeros(vocab_rows, d.shape[1], dtype=dtype)
    if tp_world > 1:
        inside = (ids >= first) & (ids < last)
        g.index_add_(0, (ids - first)[inside], d[inside])
    else:
        g.index_add_(0, ids, d)
    return g


# --------------------------------------------------------------------------------------
# vocab-parallel cross entropy.  loss.py:15-97 (forward), :99-127 (backward)
# --------------------------------------------------------------------------------------
def cross_entropy_fwd(shards, target, label_smoothing=0.0, collectives=True, ranks=None, dtype=F64):
    """shards: list over ranks of [..., partition_vocab] logits.  Returns one dict per rank with
    the reference's keys (loss, softmax, target_mask, masked_target_1d, vocab_size,
    label_smoothing) plus the row statistics (row_max, sum_exp, predicted)."""
    world = len(shards)
    ranks = list(range(world)) if ranks is None else ranks
    xs = [s.to(dtype) for s in shards]
    part = xs[0].shape[-1]

    def allreduce(vals, op):
        if not collectives:
            return vals
        red = torch.stack(vals).amax(0) if op == "max" else torch.stack(vals).sum(0)
        return [red.clone() for _ in vals]

    maxes = allreduce([x.max(-1)[0] for x in xs], "max")                          # :21-25
    xs = [x - m.unsqueeze(-1) for x, m in zip(xs, maxes)]                         # :27
    masks, mts, preds = [], [], []
    for x, r in zip(xs, ranks):
        first, last = vocab_range(part, r)                                        # :30-34
        mask = (target < first) | (target >= last)                                # :37
        mt = target.clone() - first
        mt[mask] = 0                                                              # :38-39
        x2 = x.reshape(-1, part)
        p = x2[torch.arange(x2.shape[0]), mt.reshape(-1)].clone().view_as(target).to(dtype)   # :44-49
        p[mask] = 0.0                                                             # :50
        masks.append(mask); mts.append(mt.reshape(-1)); preds.append(p)
    preds = allreduce(preds, "sum")                                               # :52-56
    exps = [torch.exp(x) for x in xs]                                             # :59-60
    sums = allreduce([e.sum(-1) for e in exps], "sum")                            # :61-66
    out = []
    for e, s, p, mask, mt, m in zip(exps, sums, preds, masks, mts, maxes):
        loss = torch.log(s) - p                                                   # :67
        sm = e / s.unsqueeze(-1)                                                  # :70
        if label_smoothing > 0:                                                   # :73-90
            smoothing = label_smoothing * part / (part - 1)
            loss = (1.0 - smoothing) * loss - smoothing * torch.log(sm).mean(-1)
        out.append({"loss": loss, "label_smoothing": label_smoothing, "vocab_size": part, "softmax": sm,
                    "target_mask": mask, "masked_target_1d": mt, "row_max": m, "sum_exp": s, "predicted": p})
    return out


def cross_entropy_bwd(fwd: dict, dout, dtype=F64):
    """loss.py:99-127: d loss / d logits of one rank, scaled by dout per row."""
    sm = fwd["softmax"].to(dtype).clone()
    part = sm.shape[-1]
    g = sm.view(-1, part)
    rows = torch.arange(g.shape[0])
    upd = 1.0 - fwd["target_mask"].view(-1).to(dtype)                              # :114
    ls, vs = fwd["label_smoothing"], fwd["vocab_size"]
    if ls > 0:                                                                    # :116-120
        smoothing = ls * vs / (vs - 1)
        g[rows, fwd["masked_target_1d"]] -= (1.0 - smoothing) * upd
        g[rows, :] -= smoothing / vs
    else:
        g[rows, fwd["masked_target_1d"]] -= upd                                   # :122
    return sm * dout.to(dtype).unsqueeze(-1)                                      # :125


# --------------------------------------------------------------------------------------
# masked mean of the per-token losses.  loss.py:131-153 (forward), :155-164 (backward)
# --------------------------------------------------------------------------------------
def mask_scale_loss_fwd(losses, loss_mask, num_microbatch=1, loss_scale=1.0, dtype=F64):
    lm = loss_mask.reshape(-1).to(dtype)
    return (losses.to(dtype).reshape(-1) * lm).sum() / lm.sum() / num_microbatch * loss_scale


def mask_scale_loss_bwd(losses, loss_mask, num_microbatch=1, loss_scale=1.0, dtype=F64):
    """d loss / d losses (the reference backpropagates a gradient of one, :156-157)."""
    lm = loss_mask.to(dtype)
    return (lm / lm.sum() / num_microbatch * loss_scale).view_as(losses)
