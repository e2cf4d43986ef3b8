"""Oracle for one pre-norm Llama decoder layer, forward and backward (autograd).

Test infrastructure: eager PyTorch on the CPU.  This is also "the PyTorch CPU eager
path" whose time is reported beside the GPU numbers.

Layer (dropout 0, no biases), following the op chain of dhellam/core/dstb.py:700-757:
  h1 = RMSNorm(x) -> [gather] -> qkv = X Wqkv^T -> RoPE(q, k) -> causal GQA attention
  -> a = o Wo^T -> [scatter] -> x2 = x + a -> h2 = RMSNorm(x2) -> [gather]
  -> u = X2 Wgu^T (gate | up) -> m = silu(gate) * up -> y = m Wd^T -> [scatter] -> out = x2 + y
QKV packing per kv group g: [q heads of g | k_g | v_g].
Sequence-parallel stand-ins (one rank's view, no cross-rank sum): gather(h, P) writes the
rank's rows into the peer tensor P and returns it, its backward returns the rank's row
slice of the incoming gradient; scatter(a, G) returns the rank's row slice, its backward
writes the slice's gradient into the peer-gradient tensor G and returns that.
"""
from __future__ import annotations

import math

import torch

from . import attention as OA
from . import ops as O


class _Gather(torch.autograd.Function):
    @staticmethod
    def forward(ctx, h, peer, r0, r1):
        ctx.r = (r0, r1)
        out = peer.clone()
        out[r0:r1] = h
        return out

    @staticmethod
    def backward(ctx, g):
        r0, r1 = ctx.r
        return g[r0:r1], None, None, None


class _Scatter(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, peer_grad, r0, r1):
        ctx.r = (r0, r1)
        ctx.save_for_backward(peer_grad)
        return a[r0:r1].clone()

    @staticmethod
    def backward(ctx, g):
        r0, r1 = ctx.r
        (pg,) = ctx.saved_tensors
        out = pg.clone()
        out[r0:r1] = g
        return out, None, None, None


def _rms(x, gamma, eps):
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * gamma


def layer_forward(cfg: dict, P: dict, x, mb: dict, dtype=torch.float64, rnd=lambda t: t):
    """Forward of the layer on x [rows, hidden] (autograd-capable).  cfg / P / mb as in ``layer_fwd_bwd``."""
    hq, hk, d, F = cfg["heads"], cfg["groups"], cfg["head_dim"], cfg["ffn"]
    b, s, tp, rk = cfg["batch"], cfg["seq"], cfg["tp"], cfg["tp_rank"]
    T = b * s
    rows = T // tp
    r0, r1 = rk * rows, (rk + 1) * rows

    def gather(h, key):
        return _Gather.apply(h, mb[key].to(dtype), r0, r1) if tp > 1 else h

    def scatter(a, key):
        return _Scatter.apply(a, mb[key].to(dtype), r0, r1) if tp > 1 else a

    h1 = rnd(_rms(x, P["ln_attn_weight"], cfg["eps"]))
    X = gather(h1, "sp_peer_attn")
    qkv = rnd(X @ P["column_attn_weight"].T)                              # [T, (hq + 2 hk) d]
    r = hq // hk
    g = qkv.view(T, hk, (r + 2) * d)
    q = g[:, :, : r * d].reshape(T, hq, d)
    k = g[:, :, r * d:(r + 1) * d]
    v = g[:, :, (r + 1) * d:]
    cp, cr = cfg.get("cp", 1), cfg.get("cp_rank", 0)
    pos = torch.arange(T) % s if cp == 1 else OA.zigzag_positions(cr, cp, s // 2).repeat(b)
    if cfg.get("theta") is not None:
        q = rnd(O.rope(q, pos, cfg["theta"], dtype=dtype))
        k = rnd(O.rope(k, pos, cfg["theta"], dtype=dtype))
    if cp > 1:
        # Context parallel: this rank's tokens are the zig-zag chunks cr and 2 cp - 1 - cr of a sequence of
        # cp * s tokens; its q rows attend to its own K/V and to the cp - 1 visiting chunks (as their owners
        # rotated them) under the causal mask of the GLOBAL positions -- what the ring steps and their merge
        # amount to (dhellam/operators/ring_attn.py:90-201).  The visiting chunks get no gradient here.
        c = s // 2
        chunks = [(k.reshape(b, 2, c, hk, d), v.reshape(b, 2, c, hk, d))]
        chunks += [(kv[0].to(dtype), kv[1].to(dtype)) for kv in mb["cp_kv_chunks"]]
        o, _ = OA.zigzag_dense(q.reshape(b, 2, c, hq, d), chunks, cr, 1.0 / math.sqrt(d), dtype=dtype)
        o = rnd(o.reshape(T, hq * d))
        return _after_attention(cfg, P, x, o, rnd, scatter, gather, F)
    qh = q.view(b, s, hq, d).permute(0, 2, 1, 3)
    kh = k.reshape(b, s, hk, d).repeat_interleave(r, dim=2).permute(0, 2, 1, 3)
    vh = v.reshape(b, s, hk, d).repeat_interleave(r, dim=2).permute(0, 2, 1, 3)
    sc = torch.matmul(qh, kh.transpose(2, 3)) / math.sqrt(d)
    sc = sc.masked_fill(torch.triu(torch.ones(s, s, dtype=torch.bool), 1), float("-inf"))
    o = rnd(torch.matmul(torch.softmax(sc, -1), vh).permute(0, 2, 1, 3).reshape(T, hq * d))
    return _after_attention(cfg, P, x, o, rnd, scatter, gather, F)


def _after_attention(cfg, P, x, o, rnd, scatter, gather, F):
    """Output projection, residual, second norm and the SwiGLU FFN (steps 6-11 of the layer)."""
    a = rnd(o @ P["linear_attn_weight"].T)
    x2 = rnd(x + scatter(a, "sp_peer_attn_bwd"))
    h2 = rnd(_rms(x2, P["ln_mlp_weight"], cfg["eps"]))
    X2 = gather(h2, "sp_peer_mlp")
    u = rnd(X2 @ P["column_mlp_weight"].T)
    m = rnd(u[:, :F] * torch.sigmoid(u[:, :F]) * u[:, F:])
    y = rnd(m @ P["linear_mlp_weight"].T)
    return rnd(x2 + scatter(y, "sp_peer_mlp_bwd"))


def layer_fwd_bwd(cfg: dict, w: dict, mb: dict, dtype=torch.float64, round_to=None):
    """cfg: hidden, heads (q heads on this rank), groups (kv heads on this rank), head_dim,
    ffn (per rank), seq, batch, tp, tp_rank, eps, theta (+ cp, cp_rank: context parallelism, seq then being the
    rank's local length and mb holding cp_kv_chunks, the cp - 1 visiting KV chunks [2, b, 2, seq/2, groups, head_dim]).  w: column_attn_weight,
    linear_attn_weight, column_mlp_weight, linear_mlp_weight, ln_attn_weight,
    ln_mlp_weight.  mb: x, dy [b, seq/tp, hidden] (+ sp_peer_* [b*seq, hidden] when tp > 1).
    ``round_to``: dtype every op's output is rounded to, and with it the gradient that comes back
    through that output (a 16-bit pipeline stores both in that type).
    Returns (out, grads) with grads = {x, ln_attn_weight, ln_mlp_weight, column_attn_weight,
    linear_attn_weight, column_mlp_weight, linear_mlp_weight}."""
    rnd = O.pipeline_round(round_to)
    b, s, tp, H = cfg["batch"], cfg["seq"], cfg["tp"], cfg["hidden"]
    rows = b * s // tp
    leaf = lambda t: t.detach().to(dtype).clone().requires_grad_()         # never the caller's own tensor
    P = {k: leaf(v) for k, v in w.items()}
    x = leaf(mb["x"].reshape(rows, H))
    dy = mb["dy"].to(dtype).reshape(rows, H)
    out = layer_forward(cfg, P, x, mb, dtype, rnd)
    (out * dy).sum().backward()
    grads = {k: v.grad for k, v in P.items()}
    grads["x"] = x.grad.view(b, rows // b, H)
    return out.detach().view(b, rows // b, H), grads


def model_fwd_bwd(cfg: dict, layers: list, word_embeddings, final_ln_weight, batches: list, loss_scale=1.0,
                  dtype=torch.float64):
    """A complete one-rank model (tp = 1): embedding -> the layers -> final RMSNorm -> logits against the
    embedding table -> cross entropy -> masked mean / number of micro-batches * loss_scale, for every
    micro-batch {"token_ids", "labels", "loss_mask"} ([b, s] each); gradients summed over the micro-batches
    (dhellam/core/dsllm.py:43-106 with dhellam/core/dshb.py:98-112).  Returns (losses, grads) with grads keyed
    word_embeddings, final_ln_weight, layers.<l>.<name>."""
    from . import head as OH
    assert cfg["tp"] == 1
    leaf = lambda t: t.detach().to(dtype).clone().requires_grad_()        # never the caller's own tensor
    table, gamma = leaf(word_embeddings), leaf(final_ln_weight)
    Ps = [{k: leaf(v) for k, v in w.items()} for w in layers]
    losses = []
    for mb in batches:
        b, s = mb["token_ids"].shape
        x = OH.word_embedding_fwd(table, mb["token_ids"]).reshape(b * s, -1)
        for P in Ps:
            x = layer_forward(cfg, P, x, {}, dtype)
        logits = _rms(x, gamma, cfg["eps"]) @ table.T
        tok = OH.cross_entropy_fwd([logits.view(b, s, -1)], mb["labels"])[0]["loss"]
        loss = OH.mask_scale_loss_fwd(tok, mb["loss_mask"], len(batches), loss_scale)
        loss.backward()
        losses.append(loss.detach())
    grads = {"word_embeddings": table.grad, "final_ln_weight": gamma.grad}
    for l, P in enumerate(Ps):
        for k, v in P.items():
            grads[f"layers.{l}.{k}"] = v.grad
    return losses, grads
