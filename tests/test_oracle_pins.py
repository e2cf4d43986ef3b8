"""Pins of the CPU oracle (no GPU).  The reference ships no golden vectors or tests, so each
oracle function is pinned against what the mathematics fixes: an independent library
routine, fp64 autograd of an independently written forward, closed-form special cases,
invariants, and brute force on tiny inputs -- chosen so that a dropped term, a wrong sign,
a swapped half or a transposed operand fails at least one of them."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attention as OA
from oracle import moe as OM
from oracle import ops as O

torch.manual_seed(0)
D = torch.float64


def rnd(*s):
    return torch.randn(*s, dtype=D)


# ---- SwiGLU ----------------------------------------------------------------------------------
def test_swiglu_forward_is_silu_gate_times_up_first_half_is_gate():
    y = rnd(5, 7, 12)
    ref = F.silu(y[..., :6]) * y[..., 6:]
    assert torch.allclose(O.swiglu_fwd(y), ref, atol=1e-14)
    # swapping the halves must NOT give the same answer
    assert not torch.allclose(O.swiglu_fwd(y), F.silu(y[..., 6:]) * y[..., :6])


def test_swiglu_backward_matches_autograd_and_special_case():
    y = rnd(4, 10).requires_grad_()
    g = rnd(4, 5)
    (F.silu(y[:, :5]) * y[:, 5:] * g).sum().backward()
    assert torch.allclose(O.swiglu_bwd(g, y.detach()), y.grad, atol=1e-13)
    # y1 = 0: out = 0, d/dy1 = g * y2 / 2, d/dy2 = 0
    y0 = torch.cat((torch.zeros(3, 4, dtype=D), rnd(3, 4)), -1)
    g0 = rnd(3, 4)
    d = O.swiglu_bwd(g0, y0)
    assert torch.allclose(d[:, :4], g0 * y0[:, 4:] / 2) and torch.all(d[:, 4:] == 0)
    assert torch.all(O.swiglu_fwd(y0) == 0)


# ---- norms -----------------------------------------------------------------------------------
@pytest.mark.parametrize("ln", [False, True])
def test_norm_forward_matches_library(ln):
    x, g, b = rnd(6, 32), rnd(32), rnd(32)
    y, mu, rs = O.norm_fwd(x, g, b if ln else None, 1e-5)
    ref = F.layer_norm(x, (32,), g, b, 1e-5) if ln else F.rms_norm(x, (32,), g, 1e-5)
    assert torch.allclose(y, ref, atol=1e-12)
    if not ln:
        assert mu is None
        y1, _, _ = O.norm_fwd(x, torch.ones(32, dtype=D), None, 0.0)
        assert torch.allclose((y1 * y1).mean(-1), torch.ones(6, dtype=D), atol=1e-12)   # unit RMS
    else:
        assert torch.allclose(mu, x.mean(-1)) and torch.allclose(rs, 1 / torch.sqrt(x.var(-1, unbiased=False) + 1e-5))


@pytest.mark.parametrize("ln", [False, True])
def test_norm_backward_matches_autograd(ln):
    x, g, b, dy = rnd(6, 32).requires_grad_(), rnd(32).requires_grad_(), rnd(32).requires_grad_(), rnd(6, 32)
    ref = F.layer_norm(x, (32,), g, b, 1e-5) if ln else F.rms_norm(x, (32,), g, 1e-5)
    (ref * dy).sum().backward()
    _, mu, rs = O.norm_fwd(x.detach(), g.detach(), b.detach() if ln else None, 1e-5)
    dx, dg, db = O.norm_bwd(dy, x.detach(), mu, rs, g.detach())
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dg, g.grad, atol=1e-12)
    if ln:
        assert torch.allclose(db, b.grad, atol=1e-12)
        assert torch.allclose(dx.sum(-1), torch.zeros(6, dtype=D), atol=1e-12)      # LayerNorm: dx sums to 0 per row
    else:
        assert db is None
    # zero-centred gamma is gamma + 1
    y0, _, _ = O.norm_fwd(x.detach(), g.detach() - 1, None, 1e-5, zero_centered_gamma=True)
    y1, _, _ = O.norm_fwd(x.detach(), g.detach(), None, 1e-5)
    assert torch.allclose(y0, y1)


# ---- RoPE ------------------------------------------------------------------------------------
def test_rope_is_complex_rotation_of_half_pairs():
    T, H, d, theta = 9, 2, 8, 10000.0
    x = rnd(T, H, d)
    pos = torch.arange(T) * 3
    out = O.rope(x, pos, theta)
    for t in range(T):
        for j in range(d // 2):
            ang = float(np.float32(pos[t].item()) * np.float32(theta ** (-2.0 * j / d)))
            z = complex(x[t, 0, j], x[t, 0, j + d // 2]) * complex(math.cos(ang), math.sin(ang))
            assert abs(out[t, 0, j].item() - z.real) < 1e-12 and abs(out[t, 0, j + d // 2].item() - z.imag) < 1e-12


def test_rope_invariants():
    x = rnd(16, 3, 32)
    pos = torch.arange(16)
    y = O.rope(x, pos, 5e5)
    assert torch.equal(y[0], x[0])                                              # position 0 is the identity
    n = lambda t: t[..., :16] ** 2 + t[..., 16:] ** 2
    assert torch.allclose(n(y), n(x), atol=1e-12)                               # per-pair norm preserved
    assert torch.allclose(O.rope(y, pos, 5e5, backward=True), x, atol=1e-12)    # inverse
    # backward is the adjoint: <rope(x), g> == <x, rope_bwd(g)>
    g = rnd(16, 3, 32)
    assert abs((y * g).sum() - (x * O.rope(g, pos, 5e5, backward=True)).sum()) < 1e-10
    # composition R(p) R(q) = R(p + q) for angles that are exact in fp32 (inv_freq_0 = 1)
    a = O.rope(O.rope(x, torch.full((16,), 3), 5e5), torch.full((16,), 4), 5e5)
    b = O.rope(x, torch.full((16,), 7), 5e5)
    assert torch.allclose(a[..., 0], b[..., 0], atol=1e-12) and torch.allclose(a[..., 16], b[..., 16], atol=1e-12)


def test_rope_inv_freq_table():
    t = O.rope_inv_freq(10000.0, 64)
    assert t.dtype == torch.float32 and t[0].item() == 1.0
    hf = 1.0 / (10000.0 ** (torch.arange(0, 64, 2).double() / 64))
    assert torch.allclose(t.double(), hf, rtol=1e-7)


# ---- residual add, legacy kernels -------------------------------------------------------------
def test_bda_and_legacy():
    x, r, b = rnd(4, 8), rnd(4, 8), rnd(4, 8)
    assert torch.equal(O.bda_fwd(x, r), x + r)
    d1, d2 = O.bda_bwd(x)
    assert torch.equal(d1, x) and torch.equal(d2, x)
    assert torch.allclose(O.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-7)
    m = (torch.rand(4, 8) > 0.5).double()
    assert torch.equal(O.bias_mask_add(x, b, r, m), m * (x + b) + r)


# ---- attention -------------------------------------------------------------------------------
def _cu(lens):
    return torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)


@pytest.mark.parametrize("causal", [True, False])
def test_attention_forward_matches_sdpa_and_logsumexp(causal):
    lens = [7, 12]
    hq, hk, d = 4, 2, 8
    q, k, v = rnd(19, hq, d), rnd(19, hk, d), rnd(19, hk, d)
    sc = 0.3
    out, lse = OA.attn_fwd(q, k, v, _cu(lens), _cu(lens), sc, causal)
    s0 = 0
    for i, n in enumerate(lens):
        qi = q[s0:s0 + n].transpose(0, 1)[None]
        ki = k[s0:s0 + n].repeat_interleave(2, 1).transpose(0, 1)[None]
        vi = v[s0:s0 + n].repeat_interleave(2, 1).transpose(0, 1)[None]
        ref = F.scaled_dot_product_attention(qi, ki, vi, is_causal=causal, scale=sc)[0].transpose(0, 1)
        assert torch.allclose(out[s0:s0 + n], ref, atol=1e-12)
        s = torch.einsum("hqd,hkd->hqk", qi[0], ki[0]) * sc
        if causal:
            s = s.masked_fill(torch.triu(torch.ones(n, n, dtype=torch.bool), 1), float("-inf"))
        assert torch.allclose(lse[i, :, :n], torch.logsumexp(s, -1), atol=1e-12)
        s0 += n


def test_attention_brute_force_tiny():
    q, k, v = rnd(3, 1, 2), rnd(3, 1, 2), rnd(3, 1, 2)
    out, lse = OA.attn_fwd(q, k, v, _cu([3]), _cu([3]), 1.0, True)
    for i in range(3):
        w = [math.exp(float(q[i, 0] @ k[j, 0])) for j in range(i + 1)]
        ref = sum(wj * v[j, 0] for j, wj in enumerate(w)) / sum(w)
        assert torch.allclose(out[i, 0], ref, atol=1e-12)
        assert abs(lse[0, 0, i].item() - math.log(sum(w))) < 1e-12


@pytest.mark.parametrize("causal,lens_q,lens_k", [(True, [6, 9], [6, 9]), (False, [5], [11])])
def test_attention_backward_matches_autograd(causal, lens_q, lens_k):
    hq, hk, d, sc = 4, 2, 8, 0.25
    tq, tk = sum(lens_q), sum(lens_k)
    q, k, v, do = rnd(tq, hq, d), rnd(tk, hk, d), rnd(tk, hk, d), rnd(tq, hq, d)
    qa, ka, va = (t.clone().requires_grad_() for t in (q, k, v))
    # independent forward for autograd: SDPA per sequence
    outs = []
    a = b = 0
    for nq, nk in zip(lens_q, lens_k):
        qi = qa[a:a + nq].transpose(0, 1)[None]
        ki = ka[b:b + nk].repeat_interleave(2, 1).transpose(0, 1)[None]
        vi = va[b:b + nk].repeat_interleave(2, 1).transpose(0, 1)[None]
        outs.append(F.scaled_dot_product_attention(qi, ki, vi, is_causal=causal, scale=sc)[0].transpose(0, 1))
        a += nq; b += nk
    (torch.cat(outs) * do).sum().backward()
    out, lse = OA.attn_fwd(q, k, v, _cu(lens_q), _cu(lens_k), sc, causal)
    dq, dk, dv, delta = OA.attn_bwd(do, q, k, v, out, lse, _cu(lens_q), _cu(lens_k), sc, causal)
    assert torch.allclose(dq, qa.grad, atol=1e-12)
    assert torch.allclose(dk, ka.grad, atol=1e-12) and torch.allclose(dv, va.grad, atol=1e-12)
    assert torch.allclose(delta[0, :, :lens_q[0]], (do * out)[:lens_q[0]].sum(-1).T, atol=1e-12)


# ---- ring step + merge ------------------------------------------------------------------------
def test_merge_properties():
    b, sq, hq, d = 1, 6, 2, 4
    o1, o2, l1, l2 = rnd(6, hq, d), rnd(6, hq, d), rnd(1, hq, 6), rnd(1, hq, 6)
    a, la = OA.merge([o1, o2], [l1, l2], [0, 0], [6, 6], b, sq, hq, d)
    c, lc = OA.merge([o2, o1], [l2, l1], [0, 0], [6, 6], b, sq, hq, d)
    assert torch.allclose(a, c) and torch.allclose(la, lc)                       # commutative
    # a partial with lse = -inf contributes nothing
    e, le = OA.merge([o1, o2], [l1, torch.full_like(l2, float("-inf"))], [0, 0], [6, 6], b, sq, hq, d)
    assert torch.allclose(e, o1) and torch.allclose(le, l1)
    # weights are a softmax over the lse values
    w = torch.softmax(torch.stack((l1, l2)), 0).transpose(2, 3)[..., None]      # [2, b, sq, hq, 1]
    assert torch.allclose(a.view(1, 6, hq, d), o1.view(1, 6, hq, d) * w[0] + o2.view(1, 6, hq, d) * w[1])


@pytest.mark.parametrize("rank", [0, 1, 2, 3])
def test_ring_equals_one_dense_causal_attention(rank):
    """The strongest pin of the ring state machine: for every rank, the merged result of the
    cp steps equals ONE dense attention over all 2*cp chunks with the causal mask taken from
    the global zig-zag positions; the ring backward equals that dense attention's autograd."""
    cp, b, c, hq, hk, d = 4, 2, 5, 4, 2, 8
    sc = 1 / math.sqrt(d)
    q = rnd(b, 2, c, hq, d)
    chunks = [(rnd(b, 2, c, hk, d), rnd(b, 2, c, hk, d)) for _ in range(cp)]
    dout = rnd(b, 2, c, hq, d)
    out, lse, steps = OA.ring_fwd(q, chunks, rank, sc)
    assert [s[0] for s in steps] == ["D"] + ["L"] * rank + ["U"] * (cp - 1 - rank)
    qa = q.clone().requires_grad_()
    ca = [(k.clone().requires_grad_(), v.clone().requires_grad_()) for k, v in chunks]
    od, ld = OA.zigzag_dense(qa, ca, rank, sc)
    assert torch.allclose(out.view(b, 2 * c, hq, d), od, atol=1e-12)
    assert torch.allclose(lse, ld, atol=1e-12)
    (od * dout.view(b, 2 * c, hq, d)).sum().backward()
    dq, dkv = OA.ring_bwd(dout, out, lse, q, chunks, rank, sc)
    assert torch.allclose(dq, qa.grad, atol=1e-12)
    for (dk, dv), (ka, va) in zip(dkv, ca):
        assert torch.allclose(dk, ka.grad, atol=1e-12) and torch.allclose(dv, va.grad, atol=1e-12)


def test_zigzag_positions():
    assert OA.zigzag_positions(1, 4, 3).tolist() == [3, 4, 5, 18, 19, 20]
    allpos = sorted(p for r in range(4) for p in OA.zigzag_positions(r, 4, 3).tolist())
    assert allpos == list(range(24))


# ---- MoE -------------------------------------------------------------------------------------
def test_route_topk_brute_force_with_ties():
    lg = np.array([[0.5, 2.0, 2.0, -1.0], [1.0, 1.0, 1.0, 1.0], [3.0, -2.0, 0.0, 3.0]], dtype=np.float32)
    idx, gates = OM.route_topk(lg, 2)
    assert idx.tolist() == [[1, 2], [0, 1], [0, 3]]                              # ties: lower expert id first
    p = torch.softmax(torch.from_numpy(lg).double(), -1)
    top, ti = torch.topk(p, 2)
    assert torch.allclose(torch.from_numpy(gates), top / top.sum(1, keepdim=True))   # renormalised top-k probs
    assert np.allclose(gates.sum(1), 1.0)


def test_sort_is_stable_bijection():
    rng = np.random.default_rng(0)
    idx = rng.integers(0, 8, size=(100, 2)).astype(np.int32)
    tpe, offs, sidx, dest = OM.sort_assignments(idx, 8)
    flat = idx.reshape(-1)
    assert tpe.sum() == 200 and offs[-1] == 200 and np.array_equal(np.diff(offs), tpe)
    assert sorted(sidx.tolist()) == list(range(200))                               # bijection
    assert np.array_equal(sidx[dest], np.arange(200))                              # dest is the inverse
    # brute force: sorted by (expert, assignment id)
    assert sidx.tolist() == [a for _, a in sorted((int(flat[a]), a) for a in range(200))]


def test_permute_unpermute_roundtrip_and_adjoint():
    rng = np.random.default_rng(1)
    T, H, E, k = 40, 6, 4, 2
    lg = rng.standard_normal((T, E)).astype(np.float32)
    idx, gates = OM.route_topk(lg, k)
    tpe, offs, sidx, dest = OM.sort_assignments(idx, E)
    x = rnd(T, H)
    xp = OM.permute(x, sidx, offs, 0, E, k)
    assert xp.shape == (T * k, H)
    # all experts local, gates renormalised to sum 1: unpermute(permute(x)) == x
    back = OM.unpermute(xp, dest, offs, 0, E, T, k, torch.from_numpy(gates))
    assert torch.allclose(back, x, atol=1e-12)
    # rows of expert e really are the tokens routed to e, in token order
    e = 2
    rows = OM.permute(x, sidx, offs, e, e + 1, k)
    toks = [t for t in range(T) for j in range(k) if idx[t, j] == e]
    assert torch.equal(rows, x[toks])
    # permute and (gate-free) unpermute are adjoint: <permute(x), y> == <x, unpermute(y)>
    y = rnd(int(offs[3] - offs[1]), H)
    lhs = (OM.permute(x, sidx, offs, 1, 3, k) * y).sum()
    rhs = (x * OM.unpermute(y, dest, offs, 1, 3, T, k, None)).sum()
    assert abs(lhs - rhs) < 1e-10
    # gate gradient by autograd
    g = torch.from_numpy(gates).clone().requires_grad_()
    dout = rnd(T, H)
    (OM.unpermute(y, dest, offs, 1, 3, T, k, g) * dout).sum().backward()
    assert torch.allclose(OM.gate_grad(dout, y, dest, offs, 1, 3, T, k), g.grad, atol=1e-12)


def test_grouped_ffn_matches_per_expert_loop():
    H, Fh = 8, 6
    x, w1, w2 = rnd(10, H), rnd(2, 2 * Fh, H), rnd(2, H, Fh)
    offs = np.array([3, 7, 13])
    y, h, a = OM.grouped_ffn(x, w1, w2, offs)
    r0 = F.silu(x[:4] @ w1[0, :Fh].T) * (x[:4] @ w1[0, Fh:].T) @ w2[0].T
    r1 = F.silu(x[4:] @ w1[1, :Fh].T) * (x[4:] @ w1[1, Fh:].T) @ w2[1].T
    assert torch.allclose(y, torch.cat((r0, r1)), atol=1e-12)


# ---- head block: embedding, vocab-parallel cross entropy, masked mean ----------------------------
from oracle import head as OH  # noqa: E402


@pytest.mark.parametrize("ls", [0.0, 0.1])
def test_cross_entropy_one_rank_is_the_library_cross_entropy(ls):
    x, t = rnd(3, 5, 11), torch.randint(0, 11, (3, 5))
    out = OH.cross_entropy_fwd([x], t, ls)[0]
    # the reference's smoothing is the library's with eps' = eps K / (K - 1)
    eps = ls * 11 / 10
    xr = x.clone().requires_grad_(True)
    ref = F.cross_entropy(xr.view(-1, 11), t.view(-1), reduction="none", label_smoothing=eps).view(3, 5)
    assert torch.allclose(out["loss"], ref, atol=1e-12)
    assert torch.allclose(out["softmax"], F.softmax(x, -1), atol=1e-14)
    dout = rnd(3, 5)
    (ref * dout).sum().backward()
    assert torch.allclose(OH.cross_entropy_bwd(out, dout), xr.grad, atol=1e-12)
    # a wrong sign on the one-hot term or a missing dout would not survive this
    assert not torch.allclose(OH.cross_entropy_bwd(out, torch.ones(3, 5)), xr.grad, atol=1e-3)


def test_cross_entropy_sharded_with_collectives_equals_unsharded():
    world, part = 4, 6
    x, t = rnd(7, world * part), torch.randint(0, world * part, (7,))
    t[0], t[1] = 0, world * part - 1                       # first id of the first rank, last id of the last
    outs = OH.cross_entropy_fwd(list(x.split(part, -1)), t)
    ref = F.cross_entropy(x, t, reduction="none")
    for r, o in enumerate(outs):
        assert torch.allclose(o["loss"], ref, atol=1e-12)
        inside = (t >= r * part) & (t < (r + 1) * part)
        assert torch.equal(o["target_mask"], ~inside)
        assert torch.equal(o["masked_target_1d"], torch.where(inside, t - r * part, torch.zeros_like(t)))
    assert torch.allclose(torch.cat([o["softmax"] for o in outs], -1), F.softmax(x, -1), atol=1e-14)
    xr = x.clone().requires_grad_(True)
    dout = rnd(7)
    (F.cross_entropy(xr, t, reduction="none") * dout).sum().backward()
    got = torch.cat([OH.cross_entropy_bwd(o, dout) for o in outs], -1)
    assert torch.allclose(got, xr.grad, atol=1e-12)


def test_cross_entropy_single_rank_share_closed_form():
    """Without the collectives a rank sees only its slice: loss = logsumexp(slice) - x[target] if the target is
    inside; otherwise the predicted logit is 0 in the max-shifted frame (loss.py:27,50), which leaves
    logsumexp(slice) - max(slice).  Smoothing averages log softmax over the SLICE (loss.py:72,86-90)."""
    part, rank = 5, 2
    x, t = rnd(6, part), torch.tensor([10, 14, 3, 12, 15, 9])      # slice of rank 2 is [10, 15)
    o = OH.cross_entropy_fwd([x], t, 0.2, collectives=False, ranks=[rank])[0]
    lse = torch.logsumexp(x, -1)
    inside = (t >= 10) & (t < 15)
    nll = lse - torch.where(inside, x[torch.arange(6), (t - 10).clamp(0, part - 1)], x.max(-1)[0])
    s = 0.2 * part / (part - 1)
    ref = (1 - s) * nll - s * (x - lse[:, None]).mean(-1)
    assert torch.allclose(o["loss"], ref, atol=1e-12)
    assert torch.equal(o["target_mask"], ~inside)
    g = OH.cross_entropy_bwd(o, torch.ones(6))
    onehot = torch.zeros(6, part, dtype=D)
    onehot[torch.arange(6)[inside], (t - 10)[inside]] = 1.0
    assert torch.allclose(g, F.softmax(x, -1) - (1 - s) * onehot - s / part, atol=1e-12)


def test_word_embedding_shards_sum_to_the_library_embedding():
    world, part, h = 3, 4, 5
    table, ids = rnd(world * part, h), torch.randint(0, world * part, (2, 9))
    ids[0, 0], ids[0, 1] = 0, world * part - 1
    outs = [OH.word_embedding_fwd(table[r * part:(r + 1) * part], ids, r, world) for r in range(world)]
    assert torch.allclose(sum(outs), F.embedding(ids, table), atol=0)
    assert torch.equal(OH.word_embedding_fwd(table, ids), F.embedding(ids, table))
    tr = table.clone().requires_grad_(True)
    dout = rnd(2, 9, h)
    (F.embedding(ids, tr) * dout).sum().backward()
    got = torch.cat([OH.word_embedding_bwd(dout, ids, part, r, world) for r in range(world)], 0)
    assert torch.allclose(got, tr.grad, atol=1e-13)
    assert torch.allclose(OH.word_embedding_bwd(dout, ids, world * part), tr.grad, atol=1e-13)


def test_masked_mean_loss_and_its_gradient():
    losses, mask = rnd(2, 6), torch.tensor([[1, 0, 1, 1, 0, 0], [0, 0, 1, 0, 1, 1]])
    ref = losses[mask.bool()].mean() / 4 * 8.0
    assert torch.allclose(OH.mask_scale_loss_fwd(losses, mask, 4, 8.0), ref, atol=1e-14)
    lr = losses.clone().requires_grad_(True)
    (lr[mask.bool()].mean() / 4 * 8.0).backward()
    assert torch.allclose(OH.mask_scale_loss_bwd(losses, mask, 4, 8.0), lr.grad, atol=1e-14)


def test_model_oracle_without_layers_is_tied_embedding_cross_entropy():
    """The composition around the layers: embedding -> RMSNorm -> logits against the same table -> masked mean
    cross entropy, gradients summed over micro-batches, checked against the library routines."""
    from oracle import layer as OL
    vocab, h, b, s = 11, 8, 2, 5
    table, gamma = rnd(vocab, h), 1 + 0.1 * rnd(h)
    batches = [{"token_ids": torch.randint(0, vocab, (b, s)), "labels": torch.randint(0, vocab, (b, s)),
                "loss_mask": torch.tensor([[1, 1, 0, 1, 1], [0, 1, 1, 1, 0]])} for _ in range(2)]
    cfg = dict(tp=1, eps=1e-5)
    losses, grads = OL.model_fwd_bwd(cfg, [], table, gamma, batches, loss_scale=4.0)
    tr, gr = table.clone().requires_grad_(True), gamma.clone().requires_grad_(True)
    for i, mb in enumerate(batches):
        x = F.embedding(mb["token_ids"], tr)
        logits = F.rms_norm(x, (h,), gr, 1e-5) @ tr.T
        tok = F.cross_entropy(logits.view(-1, vocab), mb["labels"].view(-1), reduction="none")
        loss = tok[mb["loss_mask"].view(-1).bool()].mean() / 2 * 4.0
        assert torch.allclose(losses[i], loss.detach(), atol=1e-12)
        loss.backward()
    assert torch.allclose(grads["word_embeddings"], tr.grad, atol=1e-12)
    assert torch.allclose(grads["final_ln_weight"], gr.grad, atol=1e-12)


# ---- decoder layer ---------------------------------------------------------------------------
def _angles(s, d, theta, pos=None):
    """Rotation angles as the path defines them: position times theta^(-2j/d), both factors and their product in
    fp32 (one rounding each), [s, d/2]."""
    inv = torch.tensor([theta ** (-2.0 * j / d) for j in range(d // 2)], dtype=D).float()
    pos = torch.arange(s, dtype=torch.float32) if pos is None else pos.float()
    return (pos[:, None] * inv[None, :]).to(D)


def _independent_layer(cfg, W, x, pos=None, attention=None):
    """The layer of ``oracle.layer.layer_forward`` at tp = 1, written again from library routines only
    (F.rms_norm, F.linear, F.scaled_dot_product_attention, F.silu) with its own QKV unpacking (a Python loop
    over kv groups) and its own RoPE (complex multiplication of the (j, j + d/2) pairs)."""
    hq, hk, d, F_ = cfg["heads"], cfg["groups"], cfg["head_dim"], cfg["ffn"]
    b, s, H = cfg["batch"], cfg["seq"], cfg["hidden"]
    r = hq // hk
    h1 = F.rms_norm(x, (H,), W["ln_attn_weight"], cfg["eps"])
    qkv = F.linear(h1, W["column_attn_weight"]).view(b, s, (hq + 2 * hk) * d)
    qs, ks, vs = [], [], []
    width = (r + 2) * d
    for g in range(hk):                                    # group g: [its r q heads | k_g | v_g]
        blk = qkv[..., g * width:(g + 1) * width]
        for j in range(r):
            qs.append(blk[..., j * d:(j + 1) * d])
        ks.append(blk[..., r * d:(r + 1) * d])
        vs.append(blk[..., (r + 1) * d:(r + 2) * d])
    q, k, v = torch.stack(qs, 1), torch.stack(ks, 1), torch.stack(vs, 1)           # [b, heads, s, d]

    def rotate(t):
        ang = _angles(s, d, cfg["theta"], pos)
        z = torch.complex(t[..., : d // 2], t[..., d // 2:]) * torch.polar(torch.ones_like(ang), ang)
        return torch.cat((z.real, z.imag), -1)

    q, k = rotate(q), rotate(k)
    if attention is None:
        o = F.scaled_dot_product_attention(q, k.repeat_interleave(r, 1), v.repeat_interleave(r, 1), is_causal=True)
    else:
        o = attention(q, k.repeat_interleave(r, 1), v.repeat_interleave(r, 1))
    o = o.transpose(1, 2).reshape(b * s, hq * d)
    x2 = x + F.linear(o, W["linear_attn_weight"])
    u = F.linear(F.rms_norm(x2, (H,), W["ln_mlp_weight"], cfg["eps"]), W["column_mlp_weight"])
    return x2 + F.linear(F.silu(u[:, :F_]) * u[:, F_:], W["linear_mlp_weight"])


def _layer_case(tp=1, tp_rank=0, seed=0):
    g = torch.Generator().manual_seed(seed)
    r_ = lambda *s_, std=1.0: torch.randn(*s_, generator=g, dtype=D) * std
    cfg = dict(hidden=24, heads=4, groups=2, head_dim=6, ffn=10, seq=8, batch=2, tp=tp, tp_rank=tp_rank, eps=1e-5,
               theta=10000.0)
    H, T = cfg["hidden"], cfg["batch"] * cfg["seq"]
    W = {"column_attn_weight": r_((4 + 4) * 6, H, std=0.3), "linear_attn_weight": r_(H, 24, std=0.3),
         "column_mlp_weight": r_(20, H, std=0.3), "linear_mlp_weight": r_(H, 10, std=0.3),
         "ln_attn_weight": 1 + 0.2 * r_(H), "ln_mlp_weight": 1 + 0.2 * r_(H)}
    rows = T // tp
    mb = {"x": r_(cfg["batch"], rows // cfg["batch"], H) if rows % cfg["batch"] == 0 else r_(1, rows, H),
          "dy": r_(cfg["batch"], rows // cfg["batch"], H) if rows % cfg["batch"] == 0 else r_(1, rows, H)}
    if tp > 1:
        for key in ("sp_peer_attn", "sp_peer_attn_bwd", "sp_peer_mlp", "sp_peer_mlp_bwd"):
            mb[key] = r_(T, H)
    return cfg, W, mb


def test_layer_oracle_matches_an_independently_written_layer():
    """Output and every gradient of ``layer_fwd_bwd`` (tp = 1, GQA 4 q / 2 kv heads, batch 2, so the packing per
    kv group, the per-sequence RoPE positions and the causal mask per sequence all matter) against fp64 autograd
    of ``_independent_layer``.  A swapped q/k/v block, head-major instead of group-major packing, positions that
    run over the batch, or up/gate exchanged each fail it."""
    from oracle import layer as OL
    cfg, W, mb = _layer_case()
    out, grads = OL.layer_fwd_bwd(cfg, W, mb)
    Wr = {k_: v_.clone().requires_grad_() for k_, v_ in W.items()}
    xr = mb["x"].reshape(-1, cfg["hidden"]).clone().requires_grad_()
    ref = _independent_layer(cfg, Wr, xr)
    (ref * mb["dy"].reshape(ref.shape)).sum().backward()
    assert torch.allclose(out.reshape(ref.shape), ref.detach(), rtol=1e-12, atol=1e-12)
    assert torch.allclose(grads["x"].reshape(xr.shape), xr.grad, rtol=1e-11, atol=1e-12)
    for k_ in W:
        assert torch.allclose(grads[k_], Wr[k_].grad, rtol=1e-11, atol=1e-12), k_
    # the pin must be able to fail: head-major packing ([all q | all k | all v]) is a different layer
    Wswap = dict(W)
    d, r = cfg["head_dim"], cfg["heads"] // cfg["groups"]
    idx = torch.arange((cfg["heads"] + 2 * cfg["groups"]) * d).view(cfg["groups"], (r + 2) * d)
    head_major = torch.cat((idx[:, : r * d].reshape(-1), idx[:, r * d:(r + 1) * d].reshape(-1), idx[:, (r + 1) * d:].reshape(-1)))
    Wswap["column_attn_weight"] = W["column_attn_weight"][head_major]
    out_swapped, _ = OL.layer_fwd_bwd(cfg, Wswap, mb)
    assert not torch.allclose(out_swapped, out, atol=1e-3)


@pytest.mark.parametrize("tp_rank", [0, 2, 3])
def test_layer_oracle_sequence_parallel_stand_ins(tp_rank):
    """tp = 4: the gather stand-in puts the rank's rows into the peer tensor (all other rows stay the peer's),
    its backward hands back the rank's row slice; the scatter stand-in takes the rank's row slice, its backward
    puts the slice's gradient into the peer gradient.  Checked on the layer as a whole against explicit slicing
    in ``_sp_reference`` (every op from the library), output and all gradients."""
    from oracle import layer as OL
    cfg, W, mb = _layer_case(tp=4, tp_rank=tp_rank, seed=1)
    H, T, b, s = cfg["hidden"], cfg["batch"] * cfg["seq"], cfg["batch"], cfg["seq"]
    rows = T // 4
    r0, r1 = tp_rank * rows, (tp_rank + 1) * rows
    out, grads = OL.layer_fwd_bwd(cfg, W, mb)

    Wr = {k_: v_.clone().requires_grad_() for k_, v_ in W.items()}
    xr = mb["x"].reshape(rows, H).clone().requires_grad_()
    hq, hk, d, F_ = cfg["heads"], cfg["groups"], cfg["head_dim"], cfg["ffn"]

    def put(peer, mine):                       # the peer tensor with this rank's rows replaced
        return torch.cat((peer[:r0], mine, peer[r1:]), 0)

    def take_with_peer_grad(a, peer_grad):
        # (this rank's rows of a, a scalar whose gradient is the peer gradient on all OTHER rows of a): adding
        # the scalar to the loss gives ``a`` the gradient the scatter stand-in hands back
        mask = torch.ones(T, 1, dtype=D)
        mask[r0:r1] = 0
        return a[r0:r1], (a * mask * peer_grad).sum()

    # attention half on the gathered rows, with the library pieces of _independent_layer
    h1 = F.rms_norm(xr, (H,), Wr["ln_attn_weight"], cfg["eps"])
    X = put(mb["sp_peer_attn"], h1)
    qkv = F.linear(X, Wr["column_attn_weight"]).view(b, s, -1)
    r = hq // hk
    width = (r + 2) * d
    q = torch.stack([qkv[..., g * width + j * d: g * width + (j + 1) * d] for g in range(hk) for j in range(r)], 1)
    k = torch.stack([qkv[..., g * width + r * d: g * width + (r + 1) * d] for g in range(hk)], 1)
    v = torch.stack([qkv[..., g * width + (r + 1) * d: (g + 1) * width] for g in range(hk)], 1)
    ang = _angles(s, d, cfg["theta"])
    rot = lambda t: torch.cat(((t[..., : d // 2] * ang.cos() - t[..., d // 2:] * ang.sin()),
                               (t[..., d // 2:] * ang.cos() + t[..., : d // 2] * ang.sin())), -1)
    o = F.scaled_dot_product_attention(rot(q), rot(k).repeat_interleave(r, 1), v.repeat_interleave(r, 1), is_causal=True)
    a = F.linear(o.transpose(1, 2).reshape(T, hq * d), Wr["linear_attn_weight"])
    a_sp, carry1 = take_with_peer_grad(a, mb["sp_peer_attn_bwd"])
    x2 = xr + a_sp
    X2 = put(mb["sp_peer_mlp"], F.rms_norm(x2, (H,), Wr["ln_mlp_weight"], cfg["eps"]))
    u = F.linear(X2, Wr["column_mlp_weight"])
    y = F.linear(F.silu(u[:, :F_]) * u[:, F_:], Wr["linear_mlp_weight"])
    y_sp, carry2 = take_with_peer_grad(y, mb["sp_peer_mlp_bwd"])
    ref = x2 + y_sp
    # loss: <out, dy> plus the peer gradients flowing into the rows of a and y that belong to other ranks
    ((ref * mb["dy"].reshape(rows, H)).sum() + carry1 + carry2).backward()
    assert torch.allclose(out.reshape(rows, H), ref.detach(), rtol=1e-12, atol=1e-12)
    assert torch.allclose(grads["x"].reshape(rows, H), xr.grad, rtol=1e-11, atol=1e-12)
    for k_ in W:
        assert torch.allclose(grads[k_], Wr[k_].grad, rtol=1e-11, atol=1e-12), k_


@pytest.mark.parametrize("cp,cp_rank", [(2, 0), (2, 1), (3, 1)])
def test_layer_oracle_context_parallel(cp, cp_rank):
    """cp > 1: the rank holds the zig-zag chunks cp_rank and 2 cp - 1 - cp_rank of a sequence cp times as long.
    Checked by laying the WHOLE sequence out in its natural order -- own K/V and the visiting chunks at their global
    places, the rank's q rows at theirs (zeros elsewhere) -- and calling the library's plain causal attention on
    it; the rank's rows of that result, and autograd through it, must be what the oracle layer gives."""
    from oracle import layer as OL
    cfg, W, mb = _layer_case(seed=3)
    cfg = dict(cfg, cp=cp, cp_rank=cp_rank)
    b, s, hk, d, r = cfg["batch"], cfg["seq"], cfg["groups"], cfg["head_dim"], cfg["heads"] // cfg["groups"]
    c = s // 2
    g = torch.Generator().manual_seed(9)
    mb["cp_kv_chunks"] = [torch.randn(2, b, 2, c, hk, d, generator=g, dtype=D) for _ in range(cp - 1)]
    out, grads = OL.layer_fwd_bwd(cfg, W, mb)

    chunk_of = lambda rank: (rank, 2 * cp - 1 - rank)           # global chunk numbers a rank owns
    mine = chunk_of(cp_rank)
    pos = torch.cat([torch.arange(c) + m * c for m in mine])

    def attention(q, k, v):                                     # [b, heads, s, d], already rotated, kv heads repeated
        S = 2 * cp * c
        Q = torch.zeros(b, q.shape[1], S, d, dtype=D)
        K, V = torch.zeros_like(Q), torch.zeros_like(Q)
        idx = pos
        Q = Q.index_copy(2, idx, q)
        K = K.index_copy(2, idx, k)
        V = V.index_copy(2, idx, v)
        for i, kv in enumerate(mb["cp_kv_chunks"], start=1):     # step i brings the chunk of rank (cp_rank - i) % cp
            src = chunk_of((cp_rank - i) % cp)
            for half in (0, 1):
                sl = slice(src[half] * c, (src[half] + 1) * c)
                K[:, :, sl] = kv[0][:, half].permute(0, 2, 1, 3).repeat_interleave(r, 1)
                V[:, :, sl] = kv[1][:, half].permute(0, 2, 1, 3).repeat_interleave(r, 1)
        return F.scaled_dot_product_attention(Q, K, V, is_causal=True)[:, :, idx]

    Wr = {k_: v_.clone().requires_grad_() for k_, v_ in W.items()}
    xr = mb["x"].reshape(-1, cfg["hidden"]).clone().requires_grad_()
    ref = _independent_layer(cfg, Wr, xr, pos=pos, attention=attention)
    (ref * mb["dy"].reshape(ref.shape)).sum().backward()
    assert torch.allclose(out.reshape(ref.shape), ref.detach(), rtol=1e-12, atol=1e-12)
    assert torch.allclose(grads["x"].reshape(xr.shape), xr.grad, rtol=1e-11, atol=1e-12)
    for k_ in W:
        assert torch.allclose(grads[k_], Wr[k_].grad, rtol=1e-11, atol=1e-12), k_


def test_layer_oracle_stand_in_nodes():
    """The two autograd nodes on their own: rows outside [r0, r1) of the gathered tensor are the peer's, dx is the
    row slice; the scattered tensor is the row slice and the gradient handed back is the peer gradient with the
    slice replaced."""
    from oracle.layer import _Gather, _Scatter
    h, peer, pg = rnd(3, 5).requires_grad_(), rnd(12, 5), rnd(12, 5)
    X = _Gather.apply(h, peer, 6, 9)
    assert torch.equal(X[:6], peer[:6]) and torch.equal(X[9:], peer[9:]) and torch.equal(X[6:9], h.detach())
    G = rnd(12, 5)
    X.backward(G)
    assert torch.equal(h.grad, G[6:9])
    a = rnd(12, 5).requires_grad_()
    sl = _Scatter.apply(a, pg, 6, 9)
    assert torch.equal(sl, a.detach()[6:9])
    g = rnd(3, 5)
    sl.backward(g)
    want = pg.clone()
    want[6:9] = g
    assert torch.equal(a.grad, want)


def test_pipeline_round_rounds_value_and_gradient():
    """round_to: the value handed on and the gradient handed back are both stored in the 16-bit type."""
    x = (torch.arange(16, dtype=D) / 7 + 1).requires_grad_()
    y = O.pipeline_round(torch.bfloat16)(x)
    assert torch.equal(y.detach(), x.detach().to(torch.bfloat16).to(D))
    g = torch.arange(16, dtype=D) / 11 + 1
    y.backward(g)
    assert torch.equal(x.grad, g.to(torch.bfloat16).to(D))
    assert O.pipeline_round(None)(x) is x
