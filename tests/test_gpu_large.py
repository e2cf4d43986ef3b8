"""Maximum sizes: tensors of more than 2^31 elements through the bandwidth-bound operators.

Element offsets past 2^31 (and byte offsets past 2^32) must be formed in 64 bits everywhere.  Inputs
are drawn on the GPU (a few GB each); the rows at the start, around element 2^31 and at the end go
to the CPU oracle, and where the arithmetic is exact in the run type (the add, the transpose) the
whole result is compared.  bf16; tolerance as everywhere: rel-err <= 1e-2 against the fp64 oracle.
"""
import pytest
import torch

from oracle import head as H
from oracle import ops as O
from tests.util import assert_close

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
TWO31 = 1 << 31


def _need(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * (1 << 30):
        pytest.skip(f"needs {gib} GiB of free device memory")


def _rows_to_check(rows, cols):
    """A few rows at the start, the rows that straddle element 2^31, and the last rows."""
    mid = TWO31 // cols
    pick = sorted({0, 1, 2, mid - 1, mid, mid + 1, rows - 3, rows - 2, rows - 1})
    return torch.tensor([r for r in pick if 0 <= r < rows])


def _randn(shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=BF, device="cuda")


def test_residual_add_past_2_31_elements():
    from dhellam_amd.operators.bda import bda_fwd
    _need(16)
    n = TWO31 + (1 << 20) + 8
    x, res = _randn((n,), 0), _randn((n,), 1)
    out = bda_fwd(x, res, out=torch.empty_like(x))[0]
    for lo in range(0, n, 1 << 28):                                  # exact in bf16: compare everything
        hi = min(n, lo + (1 << 28))
        assert torch.equal(out[lo:hi], x[lo:hi] + res[lo:hi]), lo


def test_swiglu_past_2_31_elements():
    from dhellam_amd.operators.swiglu import swiglu, swiglu_back
    _need(20)
    rows, f = 299_600, 3584
    assert rows * 2 * f > TWO31
    y = _randn((rows, 2 * f), 2)
    out = swiglu(y)[0]
    g = _randn((rows, f), 3)
    dy = swiglu_back(g, y)[0]
    idx = _rows_to_check(rows, 2 * f)
    idx = torch.unique(torch.cat([idx, _rows_to_check(rows, f)]))     # the boundary in the output, too
    yc, gc = y[idx.cuda()].cpu(), g[idx.cuda()].cpu()
    assert_close(out[idx.cuda()], O.swiglu_fwd(yc), BF, "swiglu")
    assert_close(dy[idx.cuda()], O.swiglu_bwd(gc, yc), BF, "swiglu bwd")


def test_norm_past_2_31_elements():
    from dhellam_amd.operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
    _need(24)
    rows, cols = (1 << 18) + 8, 8192
    assert rows * cols > TWO31
    x = _randn((rows, cols), 4)
    gamma = (1.0 + 0.1 * torch.randn(cols)).to(BF)
    y, _, rs, _ = pylayernorm_fwd(x, gamma.cuda(), None, 1e-5, 0, False, None)
    idx = _rows_to_check(rows, cols)
    xc = x[idx.cuda()].cpu()
    yo, _, rso = O.norm_fwd(xc, gamma, None, 1e-5)
    assert_close(y[idx.cuda()], yo, BF, "y")
    assert_close(rs[idx.cuda()], rso, torch.float32, "rsigma")
    del y
    dy = _randn((rows, cols), 5)
    dx, dg, _, _ = pylayernorm_bwd(dy, x, None, rs, gamma.cuda(), 0, False, None)
    dxo, _, _ = O.norm_bwd(dy[idx.cuda()].cpu(), xc, None, rs[idx.cuda()].cpu(), gamma)
    assert_close(dx[idx.cuda()], dxo, BF, "dx")
    # the weight gradient sums over every row: against the same sum formed by torch on the GPU in fp32 chunks
    ref = torch.zeros(cols, dtype=torch.float32, device="cuda")
    for lo in range(0, rows, 1 << 14):
        hi = min(rows, lo + (1 << 14))
        ref += (dy[lo:hi].float() * x[lo:hi].float() * rs[lo:hi, None]).sum(0)
    assert_close(dg, ref.cpu(), BF, "dgamma")


def test_cross_entropy_past_2_31_elements():
    from dhellam_amd.operators.loss import cross_entropy_bwd, cross_entropy_fwd
    _need(12)
    rows, cols = 16_800, 128_256
    assert rows * cols > TWO31
    logits = _randn((1, rows, cols), 6)
    g = torch.Generator(device="cpu").manual_seed(7)
    target = torch.randint(0, cols, (1, rows), generator=g)
    dout = torch.randn(1, rows, generator=g)
    inputs = {"vocab_parallel_logits": logits, "target": target.cuda()}
    out = cross_entropy_fwd(inputs, 0.0, keep_softmax=False)
    idx = _rows_to_check(rows, cols)
    xc = logits[0, idx.cuda()].cpu()
    ref = H.cross_entropy_fwd([xc], target[0, idx])[0]
    assert_close(out["loss"][0, idx.cuda()], ref["loss"], torch.float32, "loss")
    grad = cross_entropy_bwd([inputs, out], dout.cuda(), grad_out=logits)      # over the logits
    assert grad.data_ptr() == logits.data_ptr()
    assert_close(grad[0, idx.cuda()], H.cross_entropy_bwd(ref, dout[0, idx]), BF, "d logits")


def test_transpose_past_2_31_elements():
    from dhellam_amd._Clib import transpose_2d
    _need(12)
    n = 46_344
    assert n * n > TWO31 and n % 8 == 0
    src = _randn((n, n), 8)
    out = transpose_2d(src)
    for lo in range(0, n, 4096):
        hi = min(n, lo + 4096)
        assert torch.equal(out[lo:hi], src[:, lo:hi].t()), lo


def test_embedding_past_2_31_elements():
    from dhellam_amd.operators.embedding import word_embedding_fwd
    _need(8)
    tokens, hidden, vocab = (1 << 18) + 8, 8192, 1000
    table = _randn((vocab, hidden), 9)
    g = torch.Generator(device="cpu").manual_seed(10)
    ids = torch.randint(0, vocab, (1, tokens), generator=g)
    emb = word_embedding_fwd({"vocab": table, "token_ids": ids.cuda()})["word_embeddings"]
    assert emb.numel() > TWO31
    for lo in range(0, tokens, 1 << 15):
        hi = min(tokens, lo + (1 << 15))
        assert torch.equal(emb[0, lo:hi], table[ids[0, lo:hi].cuda()]), lo


def test_rope_past_2_31_elements():
    from dhellam_amd.operators.rope import rope_bwd, rope_fwd
    _need(20)
    tokens, hq, hk, d, seq = (1 << 17) + 8, 128, 8, 128, 4096
    assert tokens * hq * d > TWO31
    q, k = _randn((tokens, hq, d), 11), _randn((tokens, hk, d), 12)
    qo, ko, _ = rope_fwd(q, k, None, 5e5, seq)
    idx = _rows_to_check(tokens, hq * d)
    pos = idx % seq
    assert_close(qo[idx.cuda()], O.rope(q[idx.cuda()].cpu(), pos, 5e5), BF, "q")
    assert_close(ko[idx.cuda()], O.rope(k[idx.cuda()].cpu(), pos, 5e5), BF, "k")
    qb, _, _ = rope_bwd(q, k, None, 5e5, seq)
    assert_close(qb[idx.cuda()], O.rope(q[idx.cuda()].cpu(), pos, 5e5, backward=True), BF, "dq")


def test_moe_rows_and_grouped_gemm_past_2_31_elements():
    from dhellam_amd.operators import moe
    _need(24)
    T, K, E, H = (1 << 17) + 8, 2, 4, 8192
    R = T * K
    assert R * H > TWO31
    x = _randn((T, H), 13)
    g = torch.Generator(device="cuda").manual_seed(14)
    logits = torch.randn((T, E), generator=g, dtype=torch.float32, device="cuda")
    idx, gates, _ = moe.route_topk(logits, K)
    plan, _ = moe.sort_assignments(idx, E)
    offs = plan.expert_offsets.cpu()
    assert int(offs[-1]) == R
    perm, _ = moe.permute_fwd(x, plan, 0, E, R)
    dest = plan.dest_row.long()
    for lo in range(0, R, 1 << 15):                                   # every assignment's row is its token's row
        hi = min(R, lo + (1 << 15))
        tok = torch.arange(lo, hi, device="cuda") // K
        assert torch.equal(perm[dest[lo:hi]], x[tok]), lo
    out, _ = moe.unpermute_fwd(perm, plan, gates, 0, E)
    rows = _rows_to_check(T, H)
    ref = x[rows.cuda()].double().cpu() * gates[rows.cuda()].double().sum(1, keepdim=True).cpu()
    assert_close(out[rows.cuda()], ref, BF, "unpermute")
    del out, x
    # grouped GEMM with the same groups: c [R, 8192] is past 2^31 elements, k is small so the flops are not
    a = _randn((R, 64), 15)
    b = _randn((E, H, 64), 16) * 0.125
    c = moe.grouped_gemm_nt(a, b, plan.expert_offsets)
    rr = _rows_to_check(R, H)
    grp = torch.bucketize(rr, offs[1:].long(), right=True)
    ref = torch.stack([a[r].double().cpu() @ b[gi].double().cpu().t() for r, gi in zip(rr.tolist(), grp.tolist())])
    assert_close(c[rr.cuda()], ref, BF, "grouped gemm")
    d_a = moe.grouped_gemm_nn(c, b, plan.expert_offsets)              # [R, 8192] x [8192, 64] per group
    ref2 = torch.stack([c[r].double().cpu() @ b[gi].double().cpu() for r, gi in zip(rr.tolist(), grp.tolist())])
    assert_close(d_a[rr.cuda()], ref2, BF, "grouped gemm nn")


def test_attention_past_2_31_elements():
    """64 sequences of 4104 tokens, 64 query heads: q, out and dq hold more than 2^31 elements.  The first and
    the last sequence are compared with the same kernels run on that sequence alone (whose parity with the
    oracle the attention tests establish)."""
    from dhellam_amd import _Clib
    _need(40)
    B, S, hq, hk, d = 64, 4104, 64, 8, 128
    total = B * S
    assert total * hq * d > TWO31
    q, k, v = _randn((total, hq, d), 17), _randn((total, hk, d), 18), _randn((total, hk, d), 19)
    do = _randn((total, hq, d), 20)
    cu = torch.arange(0, total + 1, S, dtype=torch.int32, device="cuda")
    scale = d ** -0.5
    st = torch.cuda.current_stream().cuda_stream

    def run(q_, k_, v_, do_, cu_):
        r = _Clib.pymha_varlen_fwd(q_, k_, v_, cu_, cu_, S, S, 0.0, scale, True, False, 0, False)
        out, lse = r[0], r[5]
        dq, dk, dv, _ = _Clib.pymha_varlen_bwd(do_, q_, k_, v_, out, lse, cu_, cu_, S, S, 0.0, scale, True, None, False, 0,
                                               False, st)
        return out, lse, dq, dk, dv

    out, lse, dq, dk, dv = run(q, k, v, do, cu)
    cu1 = torch.tensor([0, S], dtype=torch.int32, device="cuda")
    for bi in (0, B - 1):
        sl = slice(bi * S, (bi + 1) * S)
        o1, l1, dq1, dk1, dv1 = run(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), do[sl].contiguous(), cu1)
        for name, big, one in (("out", out[sl], o1), ("lse", lse[bi], l1[0]), ("dq", dq[sl], dq1), ("dk", dk[sl], dk1),
                               ("dv", dv[sl], dv1)):
            assert_close(big, one.cpu(), BF, f"{name}[{bi}]", scale=0.1)
