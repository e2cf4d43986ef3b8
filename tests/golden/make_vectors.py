"""Writes tests/golden/vectors.npz: small known-answer vectors for the operator path.

The reference ships no golden vectors for these operators (its tests compare two
live GPU implementations), so the expected values here come from the operators'
mathematical definitions alone: numpy float64, element-by-element loops, and
central finite differences of a scalar loss for every gradient.  Neither the
oracle package nor the HIP path nor the reference is imported.  Inputs are stored
as float32 values that are exactly representable in bf16 (so every run dtype
starts from the same numbers); expected outputs are float64.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import math
import os

import numpy as np

H = 1e-5  # finite-difference step (float64; truncation + rounding error ~1e-10 relative)


def bf16_exact(a):
    """Round float32 values to the nearest bf16 (ties to even) and return them as float32."""
    u = np.asarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def rnd(rng, *shape, std=1.0):
    return bf16_exact((rng.standard_normal(shape) * std).astype(np.float32))


def fd_grad(f, x):
    """d f(x) / d x by central differences; f returns a float."""
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        old = x[i]
        x[i] = old + H
        fp = f(x)
        x[i] = old - H
        fm = f(x)
        x[i] = old
        g[i] = (fp - fm) / (2 * H)
    return g


# ---- definitions ------------------------------------------------------------------------
def norm(x, gamma, beta, eps):
    """LayerNorm (beta given) or RMSNorm (beta None), row by row."""
    y = np.zeros_like(x)
    mu = np.zeros(x.shape[0])
    rs = np.zeros(x.shape[0])
    for r in range(x.shape[0]):
        row = x[r]
        m = sum(row) / len(row) if beta is not None else 0.0
        var = sum((t - m) ** 2 for t in row) / len(row)
        mu[r] = m
        rs[r] = 1.0 / math.sqrt(var + eps)
        for c in range(len(row)):
            y[r, c] = (row[c] - m) * rs[r] * gamma[c] + (beta[c] if beta is not None else 0.0)
    return y, mu, rs


def swiglu(y):
    f = y.shape[1] // 2
    out = np.zeros((y.shape[0], f))
    for r in range(y.shape[0]):
        for c in range(f):
            g, u = y[r, c], y[r, f + c]
            out[r, c] = g / (1.0 + math.exp(-g)) * u
    return out


def rope(x, pos, theta):
    """Rotate-half: element j pairs with j + d/2; angle = fp32(pos * fp32(theta^(-2j/d)))."""
    t, h, d = x.shape
    out = np.zeros_like(x)
    for i in range(t):
        for j in range(d // 2):
            inv = np.float32(float(theta) ** (-2.0 * j / d))
            ang = float(np.float32(np.float32(pos[i]) * inv))
            c, s = math.cos(ang), math.sin(ang)
            for a in range(h):
                x1, x2 = x[i, a, j], x[i, a, j + d // 2]
                out[i, a, j] = x1 * c - x2 * s
                out[i, a, j + d // 2] = x2 * c + x1 * s
    return out


def attention(q, k, v, cu_q, cu_k, scale, causal):
    """Per sequence, per head, per query row: softmax over the allowed keys."""
    tq, hq, d = q.shape
    hk = k.shape[1]
    out = np.zeros_like(q)
    b = len(cu_q) - 1
    max_sq = max(cu_q[i + 1] - cu_q[i] for i in range(b))
    lse = np.full((b, hq, max_sq), -np.inf)
    for i in range(b):
        for h in range(hq):
            kh = h // (hq // hk)
            for r in range(cu_q[i], cu_q[i + 1]):
                nk = cu_k[i + 1] - cu_k[i]
                allowed = (r - cu_q[i] + 1) if causal else nk
                s = [scale * float(np.dot(q[r, h], k[cu_k[i] + c, kh])) for c in range(allowed)]
                m = max(s)
                z = sum(math.exp(t - m) for t in s)
                lse[i, h, r - cu_q[i]] = m + math.log(z)
                for c in range(allowed):
                    out[r, h] += math.exp(s[c] - m) / z * v[cu_k[i] + c, kh]
    return out, lse


def merge(outs, lses):
    """Combine attention over disjoint key sets: weights exp(lse_i - logsumexp_i lse_i)."""
    l = np.logaddexp.reduce(np.stack(lses), 0)                 # [b, h, s]
    o = sum(np.exp(ls - l).transpose(0, 2, 1)[..., None] * ou for ou, ls in zip(outs, lses))
    return o, l


def route_topk(logits, k):
    """softmax over experts, top-k by probability (ties to the lower index), renormalised."""
    n, e = logits.shape
    idx = np.zeros((n, k), np.int32)
    gate = np.zeros((n, k))
    for t in range(n):
        m = max(logits[t])
        p = [math.exp(x - m) for x in logits[t]]
        z = sum(p)
        p = [x / z for x in p]
        order = sorted(range(e), key=lambda j: (-p[j], j))[:k]
        s = sum(p[j] for j in order)
        for c, j in enumerate(order):
            idx[t, c] = j
            gate[t, c] = p[j] / s
    return idx, gate


def cross_entropy(x, target, label_smoothing):
    """Per row: loss = log sum exp(x) - x[target]; with label smoothing eps over K classes
    loss = (1 - a) loss - a mean(log softmax), a = eps K / (K - 1)."""
    rows, k = x.shape
    loss = np.zeros(rows)
    for r in range(rows):
        m = max(x[r])
        lse = m + math.log(sum(math.exp(t - m) for t in x[r]))
        loss[r] = lse - x[r, target[r]]
        if label_smoothing > 0:
            a = label_smoothing * k / (k - 1)
            loss[r] = (1 - a) * loss[r] - a * sum(t - lse for t in x[r]) / k
    return loss


def main():
    rng = np.random.default_rng(20240521)
    v = {}

    # normalisation, forward and backward
    x, gamma, beta, dy = rnd(rng, 6, 48), bf16_exact(1 + 0.1 * rng.standard_normal(48)), rnd(rng, 48, std=0.1), rnd(rng, 6, 48)
    for name, b in (("rms", None), ("ln", beta)):
        xd, gd, dyd = x.astype(np.float64), gamma.astype(np.float64), dy.astype(np.float64)
        bd = None if b is None else b.astype(np.float64)
        y, mu, rs = norm(xd, gd, bd, 1e-5)
        v[f"{name}_y"], v[f"{name}_mu"], v[f"{name}_rsigma"] = y, mu, rs
        v[f"{name}_dx"] = fd_grad(lambda t: float((norm(t, gd, bd, 1e-5)[0] * dyd).sum()), xd.copy())
        v[f"{name}_dgamma"] = fd_grad(lambda t: float((norm(xd, t, bd, 1e-5)[0] * dyd).sum()), gd.copy())
        if bd is not None:
            v[f"{name}_dbeta"] = fd_grad(lambda t: float((norm(xd, gd, t, 1e-5)[0] * dyd).sum()), bd.copy())
    v.update(norm_x=x, norm_gamma=gamma, norm_beta=beta, norm_dy=dy)

    # SwiGLU
    sy, sg = rnd(rng, 5, 64), rnd(rng, 5, 32)
    v.update(swiglu_in=sy, swiglu_dout=sg, swiglu_out=swiglu(sy.astype(np.float64)))
    v["swiglu_din"] = fd_grad(lambda t: float((swiglu(t) * sg).sum()), sy.astype(np.float64))

    # RoPE (Llama-3 base 5e5) on positions that are not 0..T-1
    rx = rnd(rng, 7, 3, 64)
    rpos = np.array([0, 1, 5, 4095, 4096, 17, 131071], np.int32)
    v.update(rope_x=rx, rope_pos=rpos, rope_theta=np.float64(5e5), rope_out=rope(rx.astype(np.float64), rpos, 5e5))

    # attention: two sequences, GQA 4:2, causal self-attention and non-causal cross-attention
    for name, lq, lk, causal in (("attn_causal", [5, 9], [5, 9], True), ("attn_full", [4, 6], [11, 3], False)):
        cq, ck = np.cumsum([0] + lq).astype(np.int32), np.cumsum([0] + lk).astype(np.int32)
        q, k, vv, do = rnd(rng, cq[-1], 4, 64), rnd(rng, ck[-1], 2, 64), rnd(rng, ck[-1], 2, 64), rnd(rng, cq[-1], 4, 64)
        scale = 1.0 / math.sqrt(64)
        qd, kd, vd, dod = (t.astype(np.float64) for t in (q, k, vv, do))
        out, lse = attention(qd, kd, vd, cq, ck, scale, causal)
        loss = lambda a, b, c: float((attention(a, b, c, cq, ck, scale, causal)[0] * dod).sum())
        v.update({f"{name}_q": q, f"{name}_k": k, f"{name}_v": vv, f"{name}_do": do, f"{name}_cu_q": cq,
                  f"{name}_cu_k": ck, f"{name}_out": out, f"{name}_lse": lse,
                  f"{name}_dq": fd_grad(lambda t: loss(t, kd, vd), qd.copy()),
                  f"{name}_dk": fd_grad(lambda t: loss(qd, t, vd), kd.copy()),
                  f"{name}_dv": fd_grad(lambda t: loss(qd, kd, t), vd.copy())})

    # merge: attention over keys [0:6) and [6:14) merged == attention over [0:14)
    q, k, vv = rnd(rng, 8, 2, 64), rnd(rng, 14, 2, 64), rnd(rng, 14, 2, 64)
    cq = np.array([0, 8], np.int32)
    qd, kd, vd = (t.astype(np.float64) for t in (q, k, vv))
    o1, l1 = attention(qd, kd[:6], vd[:6], cq, np.array([0, 6]), 0.125, False)
    o2, l2 = attention(qd, kd[6:], vd[6:], cq, np.array([0, 8]), 0.125, False)
    oa, la = attention(qd, kd, vd, cq, np.array([0, 14]), 0.125, False)
    om, lm = merge([o1.reshape(1, 8, 2, 64), o2.reshape(1, 8, 2, 64)], [l1, l2])
    assert np.abs(om.reshape(8, 2, 64) - oa).max() < 1e-12 and np.abs(lm - la).max() < 1e-12
    v.update(merge_o1=o1, merge_l1=l1, merge_o2=o2, merge_l2=l2, merge_out=oa, merge_lse=la)

    # routing: top-2 of 8 with exact ties in the logits
    lg = rnd(rng, 12, 8)
    lg[3, 5] = lg[3, 1]
    lg[7, :] = 0.5
    idx, gate = route_topk(lg.astype(np.float64), 2)
    v.update(route_logits=lg, route_idx=idx, route_gate=gate)

    # cross entropy over 40 classes (the tests cut the logits into 4 tensor-parallel slices of 10 and join the
    # ranks' statistics) and over 10 classes with label smoothing; gradients by finite differences of
    # sum(loss * dout).  Embedding of the slice [20, 30): a gather, and its gradient a scatter-add.
    # (drawn from their own generator so that the vectors above keep their values)
    rng2 = np.random.default_rng(977)
    cx, cd = rnd(rng2, 6, 40, std=2.0), rnd(rng2, 6)
    ct = np.array([20, 29, 5, 0, 39, 27], np.int64)
    xd, dd = cx.astype(np.float64), cd.astype(np.float64)
    v.update(ce_x=cx, ce_target=ct, ce_dout=cd, ce_loss=cross_entropy(xd, ct, 0.0),
             ce_grad=fd_grad(lambda t: float((cross_entropy(t, ct, 0.0) * dd).sum()), xd.copy()))
    sx, st = rnd(rng2, 6, 10, std=2.0), np.array([0, 9, 5, 3, 3, 7], np.int64)
    sd = sx.astype(np.float64)
    v.update(ce_ls_x=sx, ce_ls_target=st, ce_ls_loss=cross_entropy(sd, st, 0.1),
             ce_ls_grad=fd_grad(lambda t: float((cross_entropy(t, st, 0.1) * dd).sum()), sd.copy()))
    etab, eids, edo = rnd(rng2, 10, 16), np.array([[20, 3, 29, 20], [31, 25, 20, 29]], np.int64), rnd(rng2, 2, 4, 16)
    eout, egrad = np.zeros((2, 4, 16)), np.zeros((10, 16))
    for i in range(2):
        for j in range(4):
            t = eids[i, j] - 20
            if 0 <= t < 10:
                eout[i, j] = etab[t]
                egrad[t] += edo[i, j].astype(np.float64)
    v.update(emb_table=etab, emb_ids=eids, emb_dout=edo, emb_out=eout, emb_grad=egrad)

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **v)
    print(path, os.path.getsize(path), "bytes,", len(v), "arrays")


if __name__ == "__main__":
    main()
