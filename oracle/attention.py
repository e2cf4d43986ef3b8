"""Oracle for variable-length GQA attention, its backward, and the ring step + merge.

Test infrastructure (eager PyTorch on the CPU, fp64 by default).

Shapes follow the binding: q [total_q, hq, d], k/v [total_k, hk, d], cu_seqlens
int [b+1]; lse [b, hq, max_sq] (entries beyond a sequence's length are -inf).
"""
from __future__ import annotations

import torch

F64 = torch.float64


def _expand_kv(x, hq):
    """[s, hk, d] -> [s, hq, d]: kv head j serves q heads j*ratio .. (j+1)*ratio-1."""
    return x.repeat_interleave(hq // x.shape[1], dim=1)


def attn_fwd(q, k, v, cu_q, cu_k, scale, causal, dtype=F64):
    """Dense softmax attention per sequence; csrc/operators/flash_atten.cu:220-434.

    out = softmax(q k^T * scale + mask) v; lse = logsumexp of the scaled, masked
    scores (natural log).  Causal requires sq == sk per sequence (the only causal
    use in the reference: dhellam/core/dstb.py:132-136, ring_attn.py:97-102).
    """
    hq, d = q.shape[1], q.shape[2]
    b = len(cu_q) - 1
    max_sq = max(int(cu_q[i + 1] - cu_q[i]) for i in range(b)) if b else 0
    out = torch.zeros(q.shape, dtype=dtype)
    lse = torch.full((b, hq, max_sq), float("-inf"), dtype=dtype)
    for i in range(b):
        qs, qe, ks, ke = int(cu_q[i]), int(cu_q[i + 1]), int(cu_k[i]), int(cu_k[i + 1])
        sq, sk = qe - qs, ke - ks
        if sq == 0:
            continue
        qi = q[qs:qe].to(dtype).transpose(0, 1)                    # [hq, sq, d]
        ki = _expand_kv(k[ks:ke].to(dtype), hq).transpose(0, 1)    # [hq, sk, d]
        vi = _expand_kv(v[ks:ke].to(dtype), hq).transpose(0, 1)
        s = torch.matmul(qi, ki.transpose(1, 2)) * scale           # [hq, sq, sk]
        if causal:
            assert sq == sk, "causal attention is defined here for sq == sk"
            s = s.masked_fill(torch.triu(torch.ones(sq, sk, dtype=torch.bool), 1), float("-inf"))
        l = torch.logsumexp(s, -1) if sk > 0 else torch.full((hq, sq), float("-inf"), dtype=dtype)
        p = torch.exp(s - l[..., None]) if sk > 0 else s
        out[qs:qe] = torch.matmul(p, vi).transpose(0, 1) if sk > 0 else 0
        lse[i, :, :sq] = l
    return out, lse


def attn_bwd(dout, q, k, v, out, lse, cu_q, cu_k, scale, causal, dtype=F64):
    """Closed-form backward; csrc/operators/flash_atten.cu:479-757.

    P = exp(S*scale - lse); D = rowsum(dO * O); dV = P^T dO; dP = dO V^T;
    dS = P * (dP - D); dQ = dS K * scale; dK = dS^T Q * scale (summed over the q heads
    that share a kv head).  ``out`` and ``lse`` may come from a LARGER softmax than this
    q x k block (the ring step passes the merged ones, ring_attn.py:303-381); the
    formulas are then the block's share of the full gradient.
    Returns (dq, dk, dv, delta) with delta [b, hq, max_sq].
    """
    hq, hk, d = q.shape[1], k.shape[1], q.shape[2]
    r = hq // hk
    b = len(cu_q) - 1
    max_sq = lse.shape[-1]
    dq = torch.zeros(q.shape, dtype=dtype)
    dk = torch.zeros(k.shape, dtype=dtype)
    dv = torch.zeros(v.shape, dtype=dtype)
    delta = torch.zeros((b, hq, max_sq), dtype=dtype)
    for i in range(b):
        qs, qe, ks, ke = int(cu_q[i]), int(cu_q[i + 1]), int(cu_k[i]), int(cu_k[i + 1])
        sq, sk = qe - qs, ke - ks
        if sq == 0 or sk == 0:
            continue
        qi = q[qs:qe].to(dtype).transpose(0, 1)
        ki = _expand_kv(k[ks:ke].to(dtype), hq).transpose(0, 1)
        vi = _expand_kv(v[ks:ke].to(dtype), hq).transpose(0, 1)
        doi = dout[qs:qe].to(dtype).transpose(0, 1)
        oi = out[qs:qe].to(dtype).transpose(0, 1)
        s = torch.matmul(qi, ki.transpose(1, 2)) * scale
        p = torch.exp(s - lse[i, :, :sq].to(dtype)[..., None])
        if causal:
            p = p.masked_fill(torch.triu(torch.ones(sq, sk, dtype=torch.bool), 1), 0.0)
        dl = (doi * oi).sum(-1)                                    # [hq, sq]
        dp = torch.matmul(doi, vi.transpose(1, 2))
        ds = p * (dp - dl[..., None])
        dq[qs:qe] = (torch.matmul(ds, ki) * scale).transpose(0, 1)
        dk_full = (torch.matmul(ds.transpose(1, 2), qi) * scale).transpose(0, 1)   # [sk, hq, d]
        dv_full = torch.matmul(p.transpose(1, 2), doi).transpose(0, 1)
        dk[ks:ke] = dk_full.reshape(sk, hk, r, d).sum(2)
        dv[ks:ke] = dv_full.reshape(sk, hk, r, d).sum(2)
        delta[i, :, :sq] = dl
    return dq, dk, dv, delta


# --------------------------------------------------------------------------------------
# Ring / context-parallel step.  dhellam/operators/ring_attn.py.
# Local q [b, 2, c, hq, d]; chunk visiting at step i = (k, v) each [b, 2, c, hk, d], the
# KV that originated on rank (rank - i) mod cp.
# --------------------------------------------------------------------------------------
def ring_case(i: int, rank: int) -> str:
    """ring_attn.py:90-132: 'D' diagonal (causal, all rows), 'L' lower (all q x first
    half of kv), 'U' upper (second half of q x all kv)."""
    if i == 0:
        return "D"
    return "L" if i <= rank else "U"


def _cu(b, s):
    return torch.arange(0, (b + 1) * s, s, dtype=torch.int32)


def merge(outs, lses, row_begin, rows, b, sq, hq, d, dtype=F64):
    """ring_attn.py:26-40 applied as in :146-195: lse = log(sum_i exp(lse_i)) over the
    steps covering a row; out = sum_i out_i * exp(lse_i - lse).
    outs[i] [b*rows_i, hq, d], lses[i] [b, hq, rows_i]."""
    acc = torch.zeros((b, hq, sq), dtype=dtype)           # sum of exp(lse_i)
    for o, l, rb, n in zip(outs, lses, row_begin, rows):
        acc[:, :, rb:rb + n] += torch.exp(l.to(dtype))
    lse = torch.log(acc)
    out = torch.zeros((b, sq, hq, d), dtype=dtype)
    for o, l, rb, n in zip(outs, lses, row_begin, rows):
        w = torch.exp(l.to(dtype) - lse[:, :, rb:rb + n]).transpose(1, 2).unsqueeze(-1)   # [b, n, hq, 1]
        out[:, rb:rb + n] += o.to(dtype).view(b, n, hq, d) * w
    return out.view(b * sq, hq, d), lse


def ring_fwd(q, chunks, rank, scale, dtype=F64):
    """All cp steps of fa_cp_block_fwd for one rank (causal), then the merge.
    Returns (out [b*2c, hq, d], lse [b, hq, 2c], per_step) with per_step a list of
    (case, out_i, lse_i)."""
    b, _, c, hq, d = q.shape
    s = 2 * c
    per_step, outs, lses, rbs, rws = [], [], [], [], []
    for i, (k, v) in enumerate(chunks):
        case = ring_case(i, rank)
        hk = k.shape[3]
        if case == "D":
            o, l = attn_fwd(q.reshape(b * s, hq, d), k.reshape(b * s, hk, d), v.reshape(b * s, hk, d), _cu(b, s),
                            _cu(b, s), scale, True, dtype)
            rb, n = 0, s
        elif case == "L":
            o, l = attn_fwd(q.reshape(b * s, hq, d), k[:, 0].reshape(b * c, hk, d), v[:, 0].reshape(b * c, hk, d),
                            _cu(b, s), _cu(b, c), scale, False, dtype)
            rb, n = 0, s
        else:
            o, l = attn_fwd(q[:, 1].reshape(b * c, hq, d), k.reshape(b * s, hk, d), v.reshape(b * s, hk, d),
                            _cu(b, c), _cu(b, s), scale, False, dtype)
            rb, n = c, c
        per_step.append((case, o, l))
        outs.append(o); lses.append(l); rbs.append(rb); rws.append(n)
    out, lse = merge(outs, lses, rbs, rws, b, s, hq, d, dtype)
    return out, lse, per_step


def ring_bwd(dout, out, lse, q, chunks, rank, scale, dtype=F64):
    """fa_cp_block_bwd over all steps (ring_attn.py:204-411) without the exchange:
    every step uses the MERGED out and lse.  Returns dq [b, 2, c, hq, d] and, per chunk,
    (dk, dv) [b, 2, c, hk, d] (zeros in the half an 'L' step did not read)."""
    b, _, c, hq, d = q.shape
    s = 2 * c
    dout = dout.reshape(b, 2, c, hq, d)
    out = out.reshape(b, 2, c, hq, d)
    lse2 = lse.reshape(b, hq, 2, c)
    dq = torch.zeros(q.shape, dtype=dtype)
    dkv = []
    for i, (k, v) in enumerate(chunks):
        case = ring_case(i, rank)
        hk = k.shape[3]
        dk_c = torch.zeros(k.shape, dtype=dtype)
        dv_c = torch.zeros(v.shape, dtype=dtype)
        if case == "D":
            a, bk, bv, _ = attn_bwd(dout.reshape(b * s, hq, d), q.reshape(b * s, hq, d), k.reshape(b * s, hk, d),
                                    v.reshape(b * s, hk, d), out.reshape(b * s, hq, d), lse, _cu(b, s), _cu(b, s),
                                    scale, True, dtype)
            dq += a.view(b, 2, c, hq, d)
            dk_c += bk.view(b, 2, c, hk, d); dv_c += bv.view(b, 2, c, hk, d)
        elif case == "L":
            a, bk, bv, _ = attn_bwd(dout.reshape(b * s, hq, d), q.reshape(b * s, hq, d),
                                    k[:, 0].reshape(b * c, hk, d), v[:, 0].reshape(b * c, hk, d),
                                    out.reshape(b * s, hq, d), lse, _cu(b, s), _cu(b, c), scale, False, dtype)
            dq += a.view(b, 2, c, hq, d)
            dk_c[:, 0] += bk.view(b, c, hk, d); dv_c[:, 0] += bv.view(b, c, hk, d)
        else:
            a, bk, bv, _ = attn_bwd(dout[:, 1].reshape(b * c, hq, d), q[:, 1].reshape(b * c, hq, d),
                                    k.reshape(b * s, hk, d), v.reshape(b * s, hk, d),
                                    out[:, 1].reshape(b * c, hq, d), lse2[:, :, 1].contiguous(), _cu(b, c),
                                    _cu(b, s), scale, False, dtype)
            dq[:, 1] += a.view(b, c, hq, d)
            dk_c += bk.view(b, 2, c, hk, d); dv_c += bv.view(b, 2, c, hk, d)
        dkv.append((dk_c, dv_c))
    return dq, dkv


def zigzag_positions(rank, cp, c):
    """Global token positions of a rank's local [2, c] layout: chunks rank and 2cp-1-rank."""
    a = torch.arange(c)
    return torch.cat((rank * c + a, (2 * cp - 1 - rank) * c + a))


def zigzag_dense(q, chunks, rank, scale, dtype=F64):
    """ONE dense attention of the local q rows over every visiting chunk with the causal
    mask taken from GLOBAL positions.  The ring result must equal this (autograd-capable:
    pass tensors with requires_grad to get reference gradients).
    q [b, 2, c, hq, d]; returns out [b, 2c, hq, d], lse [b, hq, 2c]."""
    cp = len(chunks)
    b, _, c, hq, d = q.shape
    pos_q = zigzag_positions(rank, cp, c)
    ks, vs, pos_k = [], [], []
    for i, (k, v) in enumerate(chunks):
        src = (rank - i) % cp
        ks.append(k.reshape(b, 2 * c, -1, d)); vs.append(v.reshape(b, 2 * c, -1, d))
        pos_k.append(zigzag_positions(src, cp, c))
    K = torch.cat(ks, 1).to(dtype); V = torch.cat(vs, 1).to(dtype); pk = torch.cat(pos_k).to(q.device)
    pos_q = pos_q.to(q.device)
    Kx = K.repeat_interleave(hq // K.shape[2], dim=2).permute(0, 2, 1, 3)     # [b, hq, S, d]
    Vx = V.repeat_interleave(hq // V.shape[2], dim=2).permute(0, 2, 1, 3)
    Q = q.reshape(b, 2 * c, hq, d).to(dtype).permute(0, 2, 1, 3)
    s = torch.matmul(Q, Kx.transpose(2, 3)) * scale
    s = s.masked_fill((pk[None, :] > pos_q[:, None])[None, None], float("-inf"))
    lse = torch.logsumexp(s, -1)
    out = torch.matmul(torch.softmax(s, -1), Vx).permute(0, 2, 1, 3)
    return out, lse
