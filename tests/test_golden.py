"""Known-answer vectors (tests/golden/vectors.npz) against the oracle (CPU) and the HIP path (GPU).

The vectors were computed from the operators' definitions in numpy float64 with
finite-difference gradients by tests/golden/make_vectors.py; nothing here recomputes
them.  Inputs are bf16-exact, so fp32, bf16 and fp16 runs all start from the same
numbers.  Tolerances: the oracle (fp64) must agree to 1e-7 relative (the finite
differences are good to ~1e-9); the HIP path to 1e-5 (fp32) / 1e-2 (bf16, fp16),
index outputs bit-exact.
"""
import math
import os

import numpy as np
import pytest
import torch

from oracle import attention as OA
from oracle import head as OH
from oracle import moe as OM
from oracle import ops as O
from tests.util import assert_close, rel_err

V = np.load(os.path.join(os.path.dirname(__file__), "golden", "vectors.npz"))
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def t(name, dtype=None):
    x = torch.from_numpy(V[name])
    return x if dtype is None else x.to(dtype)


def close64(a, name, tol=1e-7):
    e = rel_err(a, t(name))
    assert e <= tol, f"{name}: rel err {e:.3e} > {tol:.0e}"


# ------------------------------------------------------------------------------------------
# CPU: the oracle reproduces the vectors
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["rms", "ln"])
def test_oracle_norm(name):
    x, g, dy = t("norm_x"), t("norm_gamma"), t("norm_dy")
    b = t("norm_beta") if name == "ln" else None
    y, mu, rs = O.norm_fwd(x, g, b, 1e-5)
    close64(y, f"{name}_y", 1e-12)
    close64(rs, f"{name}_rsigma", 1e-12)
    if b is not None:
        close64(mu, f"{name}_mu", 1e-12)
    dx, dg, db = O.norm_bwd(dy, x, mu if b is not None else None, rs, g)
    close64(dx, f"{name}_dx")
    close64(dg, f"{name}_dgamma")
    if b is not None:
        close64(db, f"{name}_dbeta")


def test_oracle_swiglu_rope():
    close64(O.swiglu_fwd(t("swiglu_in")), "swiglu_out", 1e-12)
    close64(O.swiglu_bwd(t("swiglu_dout"), t("swiglu_in")), "swiglu_din")
    close64(O.rope(t("rope_x"), t("rope_pos"), float(V["rope_theta"])), "rope_out", 1e-12)


@pytest.mark.parametrize("name,causal", [("attn_causal", True), ("attn_full", False)])
def test_oracle_attention(name, causal):
    q, k, v, do = (t(f"{name}_{s}") for s in "q k v do".split())
    cq, ck = t(f"{name}_cu_q"), t(f"{name}_cu_k")
    out, lse = OA.attn_fwd(q, k, v, cq, ck, 0.125, causal)
    close64(out, f"{name}_out", 1e-12)
    assert torch.equal(torch.isinf(lse), torch.isinf(t(f"{name}_lse")))
    fin = ~torch.isinf(lse)
    assert rel_err(lse[fin], t(f"{name}_lse")[fin]) < 1e-12
    dq, dk, dv, _ = OA.attn_bwd(do, q, k, v, out, lse, cq, ck, 0.125, causal)
    close64(dq, f"{name}_dq")
    close64(dk, f"{name}_dk")
    close64(dv, f"{name}_dv")


def test_oracle_merge_and_route():
    out, lse = OA.merge([t("merge_o1"), t("merge_o2")], [t("merge_l1"), t("merge_l2")], [0, 0], [8, 8], 1, 8, 2, 64)
    close64(out, "merge_out", 1e-12)
    close64(lse, "merge_lse", 1e-12)
    idx, gate = OM.route_topk(V["route_logits"], 2)
    assert np.array_equal(idx, V["route_idx"])
    assert np.abs(gate - V["route_gate"]).max() < 1e-12


def test_oracle_cross_entropy_and_embedding():
    # 40 classes in 4 tensor-parallel slices, joined by the oracle's explicit collectives
    outs = OH.cross_entropy_fwd(list(t("ce_x").split(10, -1)), t("ce_target"))
    for o in outs:
        close64(o["loss"], "ce_loss", 1e-12)
    close64(torch.cat([OH.cross_entropy_bwd(o, t("ce_dout")) for o in outs], -1), "ce_grad")
    # one rank, label smoothing
    o = OH.cross_entropy_fwd([t("ce_ls_x")], t("ce_ls_target"), 0.1)[0]
    close64(o["loss"], "ce_ls_loss", 1e-12)
    close64(OH.cross_entropy_bwd(o, t("ce_dout")), "ce_ls_grad")
    close64(OH.word_embedding_fwd(t("emb_table"), t("emb_ids"), 2, 4), "emb_out", 0)
    close64(OH.word_embedding_bwd(t("emb_dout"), t("emb_ids"), 10, 2, 4), "emb_grad", 1e-14)


# ------------------------------------------------------------------------------------------
# GPU: the HIP path reproduces the vectors
# ------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_cross_entropy_and_embedding(dtype):
    """The 40-class vector through FOUR ranks' kernels: each rank's statistics of its 10-column slice, joined the way
    the all-reduces of the reference join them (max of maxima, rescaled sums, summed target logits), then each
    rank's share of the gradient from the joined statistics."""
    from dhellam_amd.common import parallel_state as ps
    from dhellam_amd.operators.embedding import word_embedding_bwd, word_embedding_fwd
    from dhellam_amd.operators.loss import cross_entropy_bwd, cross_entropy_fwd
    try:
        x, tgt, dout = t("ce_x", dtype).cuda(), t("ce_target").cuda(), t("ce_dout", torch.float32).cuda()
        ctxs = []
        for r in range(4):
            ps.set_tensor_model_parallel(r, 4)
            inputs = {"vocab_parallel_logits": x[:, 10 * r:10 * r + 10].contiguous(), "target": tgt}
            ctxs.append([inputs, cross_entropy_fwd(inputs, 0.0, keep_softmax=False)])
        m = torch.stack([c[1]["row_max"] for c in ctxs])
        big = m.amax(0)
        ssum = sum(c[1]["sum_exp"] * torch.exp(c[1]["row_max"] - big) for c in ctxs)
        pred = sum(torch.where(c[1]["target_mask"], torch.zeros_like(big), c[1]["predicted"] + c[1]["row_max"] - big)
                   for c in ctxs)
        assert_close(torch.log(ssum) - pred, t("ce_loss"), torch.float32, "loss")
        grads = []
        for r, c in enumerate(ctxs):
            ps.set_tensor_model_parallel(r, 4)
            c[1]["row_max"], c[1]["sum_exp"] = big, ssum
            grads.append(cross_entropy_bwd(c, dout))
        assert_close(torch.cat(grads, -1), t("ce_grad"), dtype, "grad")
        # one rank, label smoothing, softmax kept and recomputed
        ps.set_tensor_model_parallel(0, 1)
        for keep in (True, False):
            inputs = {"vocab_parallel_logits": t("ce_ls_x", dtype).cuda(), "target": t("ce_ls_target").cuda()}
            out = cross_entropy_fwd(inputs, 0.1, keep_softmax=keep)
            assert_close(out["loss"], t("ce_ls_loss"), torch.float32, "smoothed loss")
            assert_close(cross_entropy_bwd([inputs, out], dout), t("ce_ls_grad"), dtype, "smoothed grad")
        ps.set_tensor_model_parallel(2, 4)
        table = t("emb_table", dtype).cuda()
        inputs = {"vocab": table, "token_ids": t("emb_ids").cuda()}
        out = word_embedding_fwd(inputs)
        assert torch.equal(out["word_embeddings"].double().cpu(), t("emb_out"))
        table.main_grad = torch.zeros(10, 16, dtype=torch.float32, device="cuda")
        word_embedding_bwd([inputs, out], t("emb_dout", dtype).cuda())
        assert_close(table.main_grad, t("emb_grad"), torch.float32, "embedding grad")
    finally:
        ps.set_tensor_model_parallel(0, 1)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["rms", "ln"])
def test_hip_norm(dtype, name):
    from dhellam_amd.operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
    x, g, dy = (t(n, dtype).cuda() for n in ("norm_x", "norm_gamma", "norm_dy"))
    ln = name == "ln"
    b = t("norm_beta", dtype).cuda() if ln else None
    y, mu, rs, _ = pylayernorm_fwd(x, g, b, 1e-5, 0, False, None)
    assert_close(y, t(f"{name}_y"), dtype, "y")
    assert_close(rs, t(f"{name}_rsigma"), torch.float32, "rsigma")
    mu32 = t(f"{name}_mu", torch.float32).cuda() if ln else None
    rs32 = t(f"{name}_rsigma", torch.float32).cuda()
    dx, dg, db, _ = pylayernorm_bwd(dy, x, mu32, rs32, g, 0, False, None)
    assert_close(dx, t(f"{name}_dx"), dtype, "dx")
    assert_close(dg, t(f"{name}_dgamma"), dtype, "dgamma")
    if ln:
        assert_close(db, t(f"{name}_dbeta"), dtype, "dbeta")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_swiglu_rope(dtype):
    from dhellam_amd.operators.rope import rope_fwd
    from dhellam_amd.operators.swiglu import swiglu, swiglu_back
    y, g = t("swiglu_in", dtype).cuda(), t("swiglu_dout", dtype).cuda()
    out, _ = swiglu(y)
    assert_close(out, t("swiglu_out"), dtype, "swiglu")
    din, _ = swiglu_back(g, y)
    assert_close(din, t("swiglu_din"), dtype, "swiglu_back")
    qr, _, _ = rope_fwd(t("rope_x", dtype).cuda(), None, t("rope_pos").cuda(), float(V["rope_theta"]), None)
    assert_close(qr, t("rope_out"), dtype, "rope")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,causal", [("attn_causal", True), ("attn_full", False)])
def test_hip_attention(dtype, name, causal):
    from dhellam_amd import _Clib
    q, k, v, do = (t(f"{name}_{s}", dtype).cuda() for s in "q k v do".split())
    cq, ck = t(f"{name}_cu_q").cuda(), t(f"{name}_cu_k").cuda()
    lq = np.diff(V[f"{name}_cu_q"])
    mq, mk = int(lq.max()), int(np.diff(V[f"{name}_cu_k"]).max())
    res = _Clib.pymha_varlen_fwd(q, k, v, cq, ck, mq, mk, 0.0, 1.0 / math.sqrt(64), causal, False, 0, False)
    out, lse = res[0], res[5]
    assert_close(out, t(f"{name}_out"), dtype, "out")
    for i, n in enumerate(lq):
        assert_close(lse[i, :, :n], t(f"{name}_lse")[i, :, :n], torch.float32, f"lse[{i}]")
    # backward from the exact out / lse, so the gradients are compared with the vectors alone
    out_x = t(f"{name}_out", dtype).cuda()
    lse_x = t(f"{name}_lse", torch.float32).cuda()
    dq, dk, dv, _ = _Clib.pymha_varlen_bwd(do, q, k, v, out_x, lse_x, cq, ck, mq, mk, 0.0, 1.0 / math.sqrt(64), causal,
                                           None, False, 0, False, torch.cuda.current_stream().cuda_stream)
    assert_close(dq, t(f"{name}_dq"), dtype, "dq")
    assert_close(dk, t(f"{name}_dk"), dtype, "dk")
    assert_close(dv, t(f"{name}_dv"), dtype, "dv")


@pytest.mark.gpu
def test_hip_merge_and_route():
    from dhellam_amd import _Clib
    from dhellam_amd.operators.moe import route_topk
    for dtype in (torch.float32, torch.bfloat16):
        out = torch.empty((8, 2, 64), dtype=dtype, device="cuda")
        lse = torch.empty((1, 2, 8), dtype=torch.float32, device="cuda")
        _Clib.pyattn_merge([t("merge_o1", dtype).cuda(), t("merge_o2", dtype).cuda()],
                           [t("merge_l1", torch.float32).cuda(), t("merge_l2", torch.float32).cuda()],
                           [0, 0], [8, 8], out, lse)
        assert_close(out, t("merge_out"), dtype, "merged out")
        assert_close(lse, t("merge_lse"), torch.float32, "merged lse")
    idx, gate, _ = route_topk(t("route_logits").cuda(), 2)
    assert np.array_equal(idx.cpu().numpy(), V["route_idx"])
    assert_close(gate, t("route_gate"), torch.float32, "gates")
