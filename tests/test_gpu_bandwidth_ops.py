"""GPU parity of the bandwidth-bound operators against the CPU oracle.

Each test feeds the SAME seeded tensors (already rounded to the run dtype) to the
HIP path (through the C ABI, via the reference-named wrappers) and to the oracle
in fp64.  Tolerances: rel-err <= 1e-5 (fp32), <= 1e-2 (bf16/fp16).
"""
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, randn

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,cols", [(1024, 1024), (512, 8192), (37, 256), (5, 4096), (3, 100), (2, 24576), (64, 64)])
@pytest.mark.parametrize("ln", [False, True])
def test_norm_fwd_bwd(dtype, rows, cols, ln):
    from dhellam_amd.operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
    x = randn((rows, cols), dtype, 0)
    gamma = (1.0 + 0.1 * randn((cols,), torch.float32, 1)).to(dtype)
    beta = (0.1 * randn((cols,), torch.float32, 2)).to(dtype) if ln else None
    dy = randn((rows, cols), dtype, 3)
    res = randn((rows, cols), dtype, 4)
    y, mu, rs, ms = pylayernorm_fwd(x.cuda(), gamma.cuda(), beta.cuda() if ln else None, 1e-5, 0, False, None)
    yo, muo, rso = O.norm_fwd(x, gamma, beta, 1e-5)
    assert ms == 0
    assert_close(y, yo, dtype, "y")
    assert_close(rs, rso, torch.float32, "rsigma")
    if ln:
        assert_close(mu, muo, torch.float32, "mu")
    else:
        assert mu is None
    # backward uses the oracle's statistics rounded to fp32, as the forward would hand over
    rs32 = rso.float()
    mu32 = muo.float() if ln else None
    dx, dg, db, _ = pylayernorm_bwd(dy.cuda(), x.cuda(), mu32.cuda() if ln else None, rs32.cuda(), gamma.cuda(), 0,
                                    False, None)
    dxo, dgo, dbo = O.norm_bwd(dy, x, mu32, rs32, gamma)
    assert_close(dx, dxo, dtype, "dx")
    assert_close(dg, dgo, dtype, "dgamma")
    if ln:
        assert_close(db, dbo, dtype, "dbeta")
    else:
        assert db is None
    # fused residual-gradient add and in-place accumulation of the weight gradients
    acc_g = randn((cols,), dtype, 5).cuda()
    acc_b = randn((cols,), dtype, 6).cuda() if ln else None
    acc_g0, acc_b0 = acc_g.clone(), (acc_b.clone() if ln else None)
    dx2, dg2, db2, _ = pylayernorm_bwd(dy.cuda(), x.cuda(), mu32.cuda() if ln else None, rs32.cuda(), gamma.cuda(),
                                       0, False, None, add_to_dgrad=res.cuda(), dgamma_out=acc_g, dbeta_out=acc_b)
    assert_close(dx2, dxo + res.double(), dtype, "dx+res")
    assert dg2 is acc_g
    assert_close(acc_g, dgo + acc_g0.double().cpu(), dtype, "dgamma accumulate")
    if ln:
        assert_close(acc_b, dbo + acc_b0.double().cpu(), dtype, "dbeta accumulate")


def test_norm_zero_centered_gamma_and_empty():
    from dhellam_amd.operators.layernorm import pylayernorm_fwd
    x = randn((16, 512), torch.float32, 0)
    g = 0.1 * randn((512,), torch.float32, 1)
    y, _, _, _ = pylayernorm_fwd(x.cuda(), g.cuda(), None, 1e-5, 0, True, None)
    yo, _, _ = O.norm_fwd(x, g, None, 1e-5, zero_centered_gamma=True)
    assert_close(y, yo, torch.float32)
    e = torch.empty((0, 512), device="cuda")
    y, mu, rs, _ = pylayernorm_fwd(e, g.cuda(), None, 1e-5, 0, False, None)
    assert y.shape == (0, 512) and rs.shape == (0,)


def test_norm_profiling_returns_ms():
    from dhellam_amd.operators.layernorm import pylayernorm_fwd
    x = randn((512, 8192), torch.bfloat16, 0).cuda()
    g = torch.ones(8192, dtype=torch.bfloat16, device="cuda")
    *_, ms = pylayernorm_fwd(x, g, None, 1e-5, 0, False, None, profiling=True)
    assert 0 < ms < 50


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(2, 512, 5632), (1, 4096, 7168), (7, 30), (3, 5, 2), (0, 64)])
def test_swiglu(dtype, shape):
    from dhellam_amd.operators.swiglu import swiglu, swiglu_back
    y = randn(shape, dtype, 0)
    g = randn(shape[:-1] + (shape[-1] // 2,), dtype, 1)
    out, ms = swiglu(y.cuda())
    assert ms == 0 and out.shape == g.shape
    assert_close(out, O.swiglu_fwd(y), dtype, "swiglu")
    dy, _ = swiglu_back(g.cuda().view(-1, g.shape[-1]), y.cuda().view(-1, shape[-1]))
    assert_close(dy, O.swiglu_bwd(g, y).view(-1, shape[-1]), dtype, "swiglu_back")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1 * 512 * 8192, 1000003, 7, 0])
def test_bda(dtype, n):
    from dhellam_amd.operators.bda import bda_bwd, bda_fwd
    x, r = randn((n,), dtype, 0), randn((n,), dtype, 1)
    xg = x.cuda()
    out, mask, ms = bda_fwd(xg, r.cuda())
    assert out.data_ptr() == xg.data_ptr(), "bda_fwd is in place on its input"
    assert mask is None and ms == 0
    assert_close(out, O.bda_fwd(x, r), dtype, "bda")
    dres, din, _ = bda_bwd(out, None)
    assert torch.equal(dres, out) and torch.equal(din, out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,hq,hk,d,theta,seq", [(1024, 16, 16, 64, 1e4, 512), (4096, 8, 1, 128, 5e5, None),
                                                  (33, 3, 1, 32, 1e4, None), (16, 2, 0, 16, 1e4, None)])
def test_rope(dtype, T, hq, hk, d, theta, seq):
    from dhellam_amd.operators.rope import rope_bwd, rope_fwd
    # q and k are views into one packed [T, (hq + 2 hk) * d] row, as the layer produces them
    packed = randn((T, (hq + 2 * hk) * d), dtype, 0)
    pg = packed.cuda()
    q = packed[:, : hq * d].view(T, hq, d)
    k = packed[:, hq * d: (hq + hk) * d].view(T, hk, d) if hk else None
    qg = pg[:, : hq * d].view(T, hq, d)
    kg = pg[:, hq * d: (hq + hk) * d].view(T, hk, d) if hk else None
    pos = torch.arange(T) % seq if seq else torch.arange(T)
    qr, kr, _ = rope_fwd(qg, kg, None, theta, seq)
    assert_close(qr, O.rope(q, pos, theta), dtype, "q")
    if hk:
        assert_close(kr, O.rope(k, pos, theta), dtype, "k")
    # explicit positions, backward, in place
    pos32 = pos.to(torch.int32).cuda()
    dq, dk, _ = rope_bwd(qr, kr, pos32, theta, None)
    assert_close(dq, O.rope(O.rope(q, pos, theta).to(dtype), pos, theta, backward=True), dtype, "bwd")
    # inverse rotation recovers the input up to two roundings
    assert_close(dq, q, dtype, "roundtrip")


def test_legacy_kernels():
    from dhellam_amd import _Clib
    x = randn((4096, 33), torch.float16, 0)
    o = torch.empty_like(x).cuda()
    assert _Clib.pygelu(x.cuda(), o, False) == 0
    assert_close(o, O.gelu_tanh(x), torch.float16)
    b, r = randn((4096, 33), torch.float16, 1), randn((4096, 33), torch.float16, 2)
    assert _Clib.pybda(x.cuda(), b.cuda(), r.cuda(), o, 0.0, False) == 0
    assert_close(o, O.bias_mask_add(x, b, r), torch.float16)
    s = _Clib.add_tensors(x.cuda(), b.cuda())
    assert torch.equal(s.cpu(), x + b)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols", [(8, 8), (64, 256), (72, 264), (4096, 1280), (1000, 24), (16, 4104)])
def test_transpose_2d(dtype, rows, cols):
    from dhellam_amd import _Clib
    x = randn((rows, cols), dtype, rows + cols).cuda()
    assert torch.equal(_Clib.transpose_2d(x), x.t().contiguous())
    # strided source and destination: a column block of a wider matrix into a row block of a wider one
    wide = randn((rows, cols + 16), dtype, 3).cuda()
    out = torch.full((cols, rows + 8), 7.0, dtype=dtype, device="cuda")
    _Clib.transpose_2d(wide[:, 8:8 + cols], out[:, :rows])
    assert torch.equal(out[:, :rows], wide[:, 8:8 + cols].t())
    assert bool((out[:, rows:] == 7.0).all())


def test_transpose_2d_rejects():
    from dhellam_amd import _Clib
    with pytest.raises(RuntimeError):
        _Clib.transpose_2d(torch.zeros(12, 16, dtype=torch.bfloat16, device="cuda"))     # rows not a multiple of 8
    with pytest.raises(RuntimeError):
        _Clib.transpose_2d(torch.zeros(16, 16, dtype=torch.float32, device="cuda"))      # 32-bit elements
    sq = torch.zeros(16, 16, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError):
        _Clib.transpose_2d(sq, sq)                                                        # not in place
    assert _Clib.transpose_2d(torch.zeros(0, 16, dtype=torch.bfloat16, device="cuda")).shape == (16, 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,N,K", [(1024, 1024, 3072), (512, 4096, 3080), (512, 96, 4096), (1024, 1032, 1024)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_wgrad_product(dtype, T, N, K, accumulate):
    """dW = dY^T X through both operator entry points, with and without materialised transposes."""
    from dhellam_amd import _Clib
    from dhellam_amd.operators.layernorm_column import wgrad_bwd
    dy, x = randn((T, N), dtype, 11, std=0.5), randn((T, K), dtype, 12, std=0.5)
    w0 = randn((N, K), dtype, 13)
    ref = dy.double().t() @ x.double() + (w0.double() if accumulate else 0)
    # the smaller operand is the one transposed: X when the weight has fewer inputs than outputs ("TT"), else dY ("NN")
    if dtype == torch.float32:
        want = "NT"
    elif K < N and T * K >= 1 << 20:
        want = "TT"
    elif K >= 3072 and T * N >= 1 << 20:
        want = "NN"
    else:
        want = "NT"
    assert _Clib.wgrad_layout(dy.cuda(), x.cuda()) == want
    lhs, rhs = _Clib.wgrad_operands(dy.cuda(), x.cuda())
    assert lhs.is_contiguous() == (want == "NN") and rhs.is_contiguous()
    assert torch.equal(lhs, dy.cuda().t()) and torch.equal(rhs, x.cuda())
    d = w0.clone().cuda()
    _Clib.pygemm(x.cuda(), dy.cuda(), d, None, 0, False, True, accumulate, 0, False)
    assert_close(d, ref, dtype, "pygemm wgrad")
    d2 = w0.clone().cuda() if accumulate else None
    d2, _ = wgrad_bwd(None, dy.cuda(), x.cuda(), d2, accumulate, "NT", False, 0, True, None)
    assert_close(d2, ref, dtype, "wgrad_bwd")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rope_large_positions(dtype):
    """Positions up to 2^19: the 16-bit path evaluates cos / sin with the hardware's routines after its own range
    reduction, which must keep the fraction of a revolution exact although angle / 2 pi has only 7 fractional
    bits left in fp32.  Against cos / sin in fp64 of the fp32 angle, the error is the rounding of the result."""
    from dhellam_amd.operators.rope import rope_fwd, rope_inv_freq
    T, d = 4096, 128
    inv = rope_inv_freq(5e5, d, "cuda")
    pos = (torch.arange(T, device="cuda", dtype=torch.int32) * 128 + 77)
    ang = (pos.float()[:, None] * inv[None, :]).double()
    ref = torch.cat([torch.cos(ang) - torch.sin(ang), torch.cos(ang) + torch.sin(ang)], 1)
    q, k = torch.ones(T, 2, d, device="cuda", dtype=dtype), torch.ones(T, 1, d, device="cuda", dtype=dtype)
    qo, ko, _ = rope_fwd(q, k, pos, 5e5, 0, None, False)
    ulp = {torch.float32: 2.0 ** -22, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[dtype]
    for got in (qo[:, 0], qo[:, 1], ko[:, 0]):
        assert (got.double() - ref).abs().max().item() <= 0.51 * ulp + 2e-6


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,f", [(4096, 3584), (72, 200), (8, 8), (136, 1032)])
def test_swiglu_backward_with_transposed_output(dtype, rows, f):
    """dh_swiglu_bwd_t: the same gradient as dh_swiglu_bwd, bit for bit, plus its transpose; the weight-gradient
    helper picks the transpose up from the tensor."""
    from dhellam_amd import _Clib
    from dhellam_amd.operators.swiglu import swiglu_back
    y, g = randn((rows, 2 * f), dtype, 1).cuda(), randn((rows, f), dtype, 2).cuda()
    ref, _ = swiglu_back(g, y)
    got, _ = swiglu_back(g, y, with_transposed=True)
    assert torch.equal(got, ref)
    version, gt = got._dh_rows_transposed
    assert version == got._version and gt.shape == (2 * f, rows) and torch.equal(gt, ref.t().contiguous())
    x = randn((rows, 3080), dtype, 3).cuda()                     # wide enough for the transposed layout
    if rows * 2 * f >= _Clib.WGRAD_TRANSPOSE_MIN_ELEMS:
        d1 = torch.zeros(2 * f, 3080, dtype=dtype, device="cuda")
        d2 = torch.zeros_like(d1)
        _Clib.wgrad_gemm(got, x, d1, False)                      # uses the kernel's transpose
        _Clib.wgrad_gemm(ref, x, d2, False)                      # transposes by itself
        assert torch.equal(d1, d2)
        got.mul_(2)                                              # a write to the gradient retires its transpose
        _Clib.wgrad_gemm(got, x, d1, False)
        _Clib.wgrad_gemm(ref * 2, x, d2, False)
        assert torch.equal(d1, d2)
    odd, _ = swiglu_back(g[:, : f - 4].contiguous(), torch.cat([y[:, : f - 4], y[:, f: 2 * f - 4]], 1).contiguous(),
                         with_transposed=True)                   # f not a multiple of 8: plain kernel, no transpose
    assert not hasattr(odd, "_dh_rows_transposed")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,f", [(4096, 3584), (72, 200), (8, 8), (136, 1032)])
def test_swiglu_forward_with_transposed_output(dtype, rows, f):
    """dh_swiglu_fwd_t: the same result as dh_swiglu_fwd, bit for bit, plus its transpose; the weight-gradient
    helper picks the transpose up from the tensor (the layout that hands X over transposed)."""
    from dhellam_amd import _Clib
    from dhellam_amd.operators.swiglu import swiglu
    y = randn((rows, 2 * f), dtype, 1).cuda()
    ref, _ = swiglu(y)
    got, _ = swiglu(y, with_transposed=True)
    assert torch.equal(got, ref)
    version, gt = got._dh_rows_transposed
    assert version == got._version and gt.shape == (f, rows) and torch.equal(gt, ref.t().contiguous())
    n = 2 * f + 8                                                # more outputs than inputs: X is the operand transposed
    dy = randn((rows, n), dtype, 3).cuda()
    if rows * f >= _Clib.WGRAD_TRANSPOSE_MIN_ELEMS:
        assert _Clib.wgrad_layout(dy, got) == "TT"
        d1 = torch.zeros(n, f, dtype=dtype, device="cuda")
        d2 = torch.zeros_like(d1)
        _Clib.wgrad_gemm(dy, got, d1, False)                     # uses the kernel's transpose
        _Clib.wgrad_gemm(dy, ref, d2, False)                     # transposes by itself
        assert torch.equal(d1, d2)
        assert_close(d1, dy.double().cpu().t() @ ref.double().cpu(), dtype, "wgrad through X^T")
    odd, _ = swiglu(torch.cat([y[:, : f - 4], y[:, f: 2 * f - 4]], 1).contiguous(), with_transposed=True)
    assert not hasattr(odd, "_dh_rows_transposed")              # f not a multiple of 8: plain kernel


def test_bandwidth_ops_are_deterministic():
    """Norm backward (staged column sums), SwiGLU, RoPE: two runs, same bits."""
    from dhellam_amd.operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
    from dhellam_amd.operators.swiglu import swiglu_back
    dt = torch.bfloat16
    x, g, dy = randn((4096, 8192), dt, 1).cuda(), randn((8192,), dt, 2).cuda(), randn((4096, 8192), dt, 3).cuda()
    _, _, rs, _ = pylayernorm_fwd(x, g, None, 1e-5, 0, False, None)
    a = pylayernorm_bwd(dy, x, None, rs, g, 0, False, None)
    b = pylayernorm_bwd(dy, x, None, rs, g, 0, False, None)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    y, gg = randn((4096, 7168), dt, 4).cuda(), randn((4096, 3584), dt, 5).cuda()
    assert torch.equal(swiglu_back(gg, y)[0], swiglu_back(gg, y)[0])


def test_binding_level_names_for_the_added_operators():
    """The `_Clib` names of the operators the reference lacks forward to the operator layer: same results, lists
    with the elapsed time appended only when profiling."""
    from dhellam_amd import _Clib
    from dhellam_amd.operators import moe
    from dhellam_amd.operators.layernorm import pylayernorm_fwd
    from dhellam_amd.operators.swiglu import swiglu
    dt = torch.bfloat16
    x, g = randn((64, 256), dt, 1).cuda(), randn((256,), dt, 2).cuda()
    out, rs = _Clib.pyrmsnorm_fwd(x, g, 1e-5, False)
    ref = pylayernorm_fwd(x, g, None, 1e-5, 0, False, None)
    assert torch.equal(out, ref[0]) and torch.equal(rs, ref[2])
    res = _Clib.pyrmsnorm_bwd(out, x, rs, g, True)
    assert len(res) == 3 and res[2] >= 0 and res[0].shape == x.shape and res[1].shape == g.shape
    q, k = randn((32, 4, 64), dt, 3).cuda(), randn((32, 2, 64), dt, 4).cuda()
    qr, kr = _Clib.pyrope_fwd(q, k, None, 1e4, False)
    q2, k2 = _Clib.pyrope_bwd(qr, kr, None, 1e4, False)
    assert_close(q2, q.cpu(), dt, "rope inverse") and assert_close(k2, k.cpu(), dt, "rope inverse")
    y = randn((64, 512), dt, 5).cuda()
    (a,) = _Clib.pyswiglu_fwd(y, False)
    assert torch.equal(a, swiglu(y)[0])
    (dy,) = _Clib.pyswiglu_bwd(a, y, False)
    assert dy.shape == y.shape
    logits = randn((128, 8), torch.float32, 6).cuda()
    idx, gates = _Clib.pymoe_route_topk(logits, 2, False)
    (plan,) = _Clib.pymoe_sort(idx, 8, False)
    rows = int(plan.expert_offsets[8].item())
    h = randn((128, 64), dt, 7).cuda()
    (xp,) = _Clib.pymoe_permute(h, plan, 0, 8, rows, False)
    (back,) = _Clib.pymoe_unpermute(xp, plan, gates, 0, 8, False)
    assert_close(back, h.cpu(), dt, "permute -> unpermute with gates summing to one")
    w = randn((8, 32, 64), dt, 8).cuda()
    c = _Clib.pygrouped_gemm_nt(xp, w, plan.expert_offsets)
    assert torch.equal(c, moe.grouped_gemm_nt(xp, w, plan.expert_offsets))
    lg, tg = randn((16, 100), dt, 9).cuda(), torch.arange(16, device="cuda") % 100
    ce = _Clib.pycross_entropy_fwd(lg, tg, 0.0, False)
    gr = _Clib.pycross_entropy_bwd(lg, tg, ce, torch.ones(16, device="cuda"))
    assert ce["loss"].shape == (16,) and gr.shape == lg.shape
    table = randn((100, 64), dt, 10).cuda()
    assert torch.equal(_Clib.pyembedding_fwd(table, tg), table[tg])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t,n,k", [(256, 384, 512), (100, 72, 40), (1, 8, 8), (4096, 1280, 1024)])
def test_dense_gemm_layouts(dtype, t, n, k):
    """pygemm (csrc/operators/gemm.cu:3-170) in its three layouts and the wrappers of
    dhellam/operators/layernorm_column.py on the same products, against fp64 matmul."""
    from dhellam_amd import _Clib
    from dhellam_amd.operators.layernorm_column import dgrad_bwd, gemm_fwd, wgrad_bwd
    x, w, dy = randn((t, k), dtype, 0), randn((n, k), dtype, 1, std=0.1), randn((t, n), dtype, 2)
    acc0 = randn((n, k), dtype, 3)
    xg, wg, dyg = x.cuda(), w.cuda(), dy.cuda()
    ref_y, ref_dx = x.double() @ w.double().t(), dy.double() @ w.double()
    ref_dw = dy.double().t() @ x.double()
    y = torch.empty(t, n, dtype=dtype, device="cuda")
    assert _Clib.pygemm(wg, xg, y, None, 0, True, False, False, 0, False) == 0.0
    assert_close(y, ref_y, dtype, "TN")
    dx = torch.empty(t, k, dtype=dtype, device="cuda")
    ms = _Clib.pygemm(wg, dyg, dx, None, 0, False, False, False, 0, True)
    assert ms > 0.0
    assert_close(dx, ref_dx, dtype, "NN")
    ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")        # the caller's workspace
    for accumulate in (False, True):
        dw = acc0.clone().cuda()
        _Clib.pygemm(xg, dyg, dw, ws, ws.numel(), False, True, accumulate, 0, False)
        assert_close(dw, ref_dw + (acc0.double() if accumulate else 0), dtype, "NT")
    # the wrappers: leading dimensions, a given output, accumulation into an fp32 gradient
    y3, _ = gemm_fwd(None, xg.view(1, t, k), wg, None, "TN", False, 0, True, None)
    assert y3.shape == (1, t, n) and torch.equal(y3.view(t, n), y)
    y4, _ = gemm_fwd(None, xg, wg, None, "TN", False, 0, False, None)
    assert torch.equal(y4, y)
    dx2, _ = dgrad_bwd(None, dyg, wg, None, "NN", False, 0, True, None)
    assert torch.equal(dx2, dx)
    g32 = acc0.float().cuda()
    out, _ = wgrad_bwd(None, dyg, xg, g32, True, "NT", False, 0, True, None)
    assert out is g32
    assert_close(g32, ref_dw + acc0.double(), torch.float32 if dtype == torch.float32 else dtype, "fp32 dW", scale=0.1 if dtype != torch.float32 else 1)
    fresh, _ = wgrad_bwd(None, dyg, xg, None, False, "NT", False, 0, True, None)
    assert_close(fresh, ref_dw, dtype, "fresh dW")
    # operands the C entry point does not take still work through the wrapper (strided view of the weight)
    wide = torch.cat([wg, wg], 1)[:, :k]
    assert not wide.is_contiguous() or k == wide.stride(0)
    y5, _ = gemm_fwd(None, xg, wide, None, "TN", False, 0, True, None)
    assert_close(y5, ref_y, dtype, "strided weight")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,n,k", [(256, 384, 512), (4096, 1280, 1024), (100, 72, 40)])
def test_dgrad_against_resident_transpose(dtype, t, n, k):
    """A weight registered with keep_transposed: the data gradient runs against W^T in the forward's layout and equals
    the NN product; the copy follows the weight through in-place updates (version counter), is usable from another
    stream, and an explicit refresh covers writers that go around the counter."""
    from dhellam_amd import _Clib
    from dhellam_amd.operators.layernorm_column import dgrad_bwd
    w, dy = randn((n, k), dtype, 1, std=0.1).cuda(), randn((t, n), dtype, 2).cuda()
    plain, _ = dgrad_bwd(None, dy, w, None, "NN", False, 0, True, None)           # not registered: NN as given
    assert _Clib.transposed_of(w) is None
    assert_close(plain, dy.double().cpu() @ w.double().cpu(), dtype, "NN")
    wt = _Clib.keep_transposed(w)
    assert torch.equal(wt, w.t().contiguous()) and _Clib.transposed_of(w) is wt
    for is_matmul in (True, False):
        got, _ = dgrad_bwd(None, dy, w, None, "NN", False, 0, is_matmul, None)
        assert_close(got, dy.double().cpu() @ w.double().cpu(), dtype, "against W^T")
        assert_close(got, plain.double().cpu(), dtype, "both layouts agree")
    w.mul_(0.5)                                                                   # an optimizer step: version moves
    got, _ = dgrad_bwd(None, dy, w, None, "NN", False, 0, True, None)
    assert torch.equal(_Clib.transposed_of(w), w.t().contiguous())
    assert_close(got, dy.double().cpu() @ w.double().cpu(), dtype, "after an in-place update")
    w.data.copy_(randn((n, k), dtype, 3, std=0.1))                                # around the counter: caller refreshes
    _Clib.keep_transposed(w, refresh=True)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):                                                 # another stream than the one that built it
        got, _ = dgrad_bwd(None, dy, w, None, "NN", False, 0, True, None)
    side.synchronize()
    assert_close(got, dy.double().cpu() @ w.double().cpu(), dtype, "from another stream")
    odd = randn((n, k + 4), dtype, 4).cuda()[:, :k]                               # not a tensor the transpose takes
    assert _Clib.keep_transposed(odd) is None and _Clib.transposed_of(odd) is None


def test_dense_gemm_argument_errors():
    import ctypes
    from dhellam_amd import _Clib, _lib
    lib = _lib.load()
    a = torch.zeros(16, 32, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(8, 32, dtype=torch.bfloat16, device="cuda")
    d = torch.zeros(8, 16, dtype=torch.bfloat16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream

    def call(ar, ac, br, bc, ta, tb, dt=1, odt=1, ws=None, wsb=0, acc=0):
        return lib.dh_gemm(a.data_ptr(), b.data_ptr(), d.data_ptr(), ar, ac, br, bc, ta, tb, acc, dt, odt, ws, wsb, st)

    assert call(16, 32, 8, 32, 1, 0) == 0                                  # TN, no workspace
    for bad in (call(16, 32, 8, 32, 1, 1),                                # TT: refused here as in the reference
                call(16, 32, 8, 24, 1, 0),                                # inner sizes differ
                call(16, 32, 8, 32, 1, 0, dt=7, odt=7),                   # unknown type
                call(16, 32, 8, 32, 1, 0, dt=1, odt=2),                   # bf16 operands, fp16 result
                call(16, 32, 8, 32, 1, 0, ws=None, wsb=1024),             # a size without a buffer
                call(16, 0, 8, 0, 1, 0)):                                 # empty sum, not accumulating
        assert bad < 0
        assert len(_lib.load().dh_last_error()) > 0
    assert call(16, 0, 8, 0, 1, 0, acc=1) == 0                            # empty sum, accumulating: nothing to do
    assert call(0, 32, 8, 32, 1, 0) == 0                                  # empty result
    with pytest.raises(RuntimeError):
        _Clib.dense_gemm(a, b, torch.zeros(16, 8, dtype=torch.bfloat16, device="cuda"), True, False, False)   # D is [n, m]
    with pytest.raises(RuntimeError):
        _Clib.dense_gemm(a, b.float(), d, True, False, False)


def test_dense_gemm_on_two_streams():
    """Products issued on two streams at once (each stream has its own library workspace) give the bits of the
    same products issued alone."""
    from dhellam_amd import _Clib
    dtype = torch.bfloat16
    x, w = randn((2048, 4096), dtype, 0).cuda(), randn((1280, 4096), dtype, 1, std=0.1).cuda()      # under-filled grid
    x2, w2 = randn((2048, 1024), dtype, 2).cuda(), randn((4096, 1024), dtype, 3, std=0.1).cuda()
    y_ref, y2_ref = torch.empty(2048, 1280, dtype=dtype, device="cuda"), torch.empty(2048, 4096, dtype=dtype, device="cuda")
    _Clib.dense_gemm(w, x, y_ref, True, False, False)
    _Clib.dense_gemm(w2, x2, y2_ref, True, False, False)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    y, y2 = torch.empty_like(y_ref), torch.empty_like(y2_ref)
    for _ in range(50):
        y.zero_(), y2.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(s1):
            _Clib.dense_gemm(w, x, y, True, False, False)
        with torch.cuda.stream(s2):
            _Clib.dense_gemm(w2, x2, y2, True, False, False)
        torch.cuda.synchronize()
        assert torch.equal(y, y_ref) and torch.equal(y2, y2_ref)
    assert len({k for k in _Clib._gemm_ws if k[1] in (s1.cuda_stream, s2.cuda_stream)}) == 2


def test_math_sm_count_confines_a_launch_to_that_many_compute_units():
    """``math_sm_count`` of the reference's bindings (libsmctrl mask, csrc/operators/gemm.cu:20-21,66-70,108;
    flash_atten.cu:248-249,407) maps to a stream with a compute-unit mask: same bits as the unconfined launch, a
    longer run on a sixteenth of the GPU, negative counts take the units from the other end, counts beyond the
    device are refused."""
    from dhellam_amd import _Clib
    n_cus = torch.cuda.get_device_properties(0).multi_processor_count
    dt = torch.bfloat16
    a, b = randn((2048, 4096), dt, 1, 0.1).cuda(), randn((4096, 4096), dt, 2, 0.1).cuda()     # weight [N, K], input [T, K]
    outs, ms = [], []
    for count in (0, n_cus // 16, -(n_cus // 16)):
        d = torch.empty((4096, 2048), dtype=dt, device="cuda")
        _Clib.pygemm(a, b, d, None, 0, True, False, False, count, False)                       # warm-up (stream creation)
        t = [_Clib.pygemm(a, b, d, None, 0, True, False, False, count, True) for _ in range(5)]
        outs.append(d)
        ms.append(sorted(t)[2])
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert ms[1] > 3 * ms[0] and ms[2] > 3 * ms[0], ms
    with pytest.raises(RuntimeError):
        _Clib.pygemm(a, b, outs[0], None, 0, True, False, False, n_cus + 1, False)
    # attention forward and backward on a quarter of the GPU: same bits
    T, hq, hk, dd = 1024, 8, 2, 128
    q, k, v, do = (randn((T, h, dd), dt, s).cuda() for h, s in ((hq, 3), (hk, 4), (hk, 5), (hq, 6)))
    cu = torch.tensor([0, T], dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    res = []
    for count in (0, n_cus // 4):
        r = _Clib.pymha_varlen_fwd(q, k, v, cu, cu, T, T, 0.0, dd ** -0.5, True, False, count, False)
        g = _Clib.pymha_varlen_bwd(do, q, k, v, r[0], r[5], cu, cu, T, T, 0.0, dd ** -0.5, True, None, False, count, False, st)
        torch.cuda.synchronize()
        res.append([r[0], r[5]] + g[:4])
    for x, y in zip(*res):
        assert torch.equal(x, y)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,cols,ln", [(512, 8192, False), (37, 1000, True), (300, 4104, False), (64, 16384, True), (5, 99, False)])
def test_residual_add_fused_into_norm_is_the_two_ops_bit_for_bit(dtype, rows, cols, ln):
    """dh_add_norm_fwd = the bda residual add followed by the norm: same sum, same normalised rows, same statistics,
    bit for bit (and therefore the oracle's, at the operators' tolerance)."""
    from dhellam_amd.operators.bda import bda_fwd
    from dhellam_amd.operators.layernorm import pylayernorm_fwd
    x, r = randn((rows, cols), dtype, 1).cuda(), randn((rows, cols), dtype, 2).cuda()
    g = (1 + 0.1 * randn((cols,), torch.float32, 3)).to(dtype).cuda()
    b = (0.1 * randn((cols,), torch.float32, 4)).to(dtype).cuda() if ln else None
    s_ref, _, _ = bda_fwd(x, r, out=torch.empty_like(x))
    y_ref, mu_ref, rs_ref, _ = pylayernorm_fwd(s_ref, g, b, 1e-5, 0, False, None)
    y, mu, rs, _, s = pylayernorm_fwd(x, g, b, 1e-5, 0, False, None, residual=r)
    assert torch.equal(s, s_ref) and torch.equal(y, y_ref) and torch.equal(rs, rs_ref)
    if ln:
        assert torch.equal(mu, mu_ref)
    yo, _, rso = O.norm_fwd(x.cpu().double() + r.cpu().double() if dtype == torch.float32 else s_ref.cpu(), g.cpu(),
                            b.cpu() if ln else None, 1e-5)
    assert_close(y, yo, dtype, "fused add + norm")
    # in place on the input, as the reference's bda is
    x2 = x.clone()
    y2, _, _, _, s2 = pylayernorm_fwd(x2, g, b, 1e-5, 0, False, None, residual=r, sum_out=x2)
    assert s2 is x2 and torch.equal(x2, s_ref) and torch.equal(y2, y_ref)


def test_reused_swiglu_gradient_buffer_drops_the_transposed_twin():
    """``swiglu_back(..., with_transposed=True)`` hangs dY^T on its result for the weight-gradient GEMM.  The
    library's kernels write through raw pointers, so the tensor's version counter does not move when the same buffer
    is written again by the plain kernel: the stale twin must be dropped, or ``wgrad_gemm`` multiplies the old one."""
    from dhellam_amd import _Clib
    from dhellam_amd.operators.swiglu import swiglu_back
    dtype, rows, f, k = torch.bfloat16, 4096, 512, 4096
    y1, g1, y2, g2 = (randn(s, dtype, i).cuda() for i, s in enumerate(((rows, 2 * f), (rows, f), (rows, 2 * f), (rows, f))))
    x = randn((rows, k), dtype, 9).cuda()
    buf = torch.empty_like(y1)
    d1, _ = swiglu_back(g1, y1, buf, None, False, with_transposed=True)
    assert d1 is buf and torch.equal(buf._dh_rows_transposed[1], buf.t().contiguous())
    assert _Clib.wgrad_layout(buf, x) == "NN"                  # the layout that picks the twin up
    d2, _ = swiglu_back(g2, y2, buf, None, False, with_transposed=False)
    assert d2 is buf and not hasattr(buf, "_dh_rows_transposed")
    out = torch.empty((2 * f, k), dtype=dtype, device="cuda")
    _Clib.wgrad_gemm(buf, x, out, False)
    assert_close(out, (buf.double().t() @ x.double()).cpu(), dtype, "wgrad of the rewritten buffer")
