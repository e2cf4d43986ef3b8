"""GPU parity of flash attention (fwd, bwd), the merge and the ring step against the oracle.

All calls go through the C ABI via the reference-named shims (pymha_varlen_fwd/bwd,
fa_cp_block_fwd/bwd).  Inputs are seeded N(0,1), rounded to the run dtype and fed
identically to the HIP path and to the oracle.  Tolerances: rel-err <= 1e-2
(bf16/fp16), <= 1e-5 (fp32) on outputs and gradients.
"""
import math

import pytest
import torch

from oracle import attention as OA
from tests.util import assert_close, randn

pytestmark = pytest.mark.gpu


def _cu(lens):
    c = [0]
    for n in lens:
        c.append(c[-1] + n)
    return torch.tensor(c, dtype=torch.int32)


def _run_fwd_bwd(dtype, lens_q, lens_k, hq, hk, d, causal, oracle_dtype=torch.float64, packed=False, seed=0):
    from dhellam_amd import _Clib
    cq, ck = _cu(lens_q), _cu(lens_k)
    tq, tk = int(cq[-1]), int(ck[-1])
    scale = 1.0 / math.sqrt(d)
    if packed:
        # q, k, v as strided views of one [T, (hq + 2 hk) d] projection output (self-attention only)
        assert tq == tk
        qkv = randn((tq, (hq + 2 * hk) * d), dtype, seed)
        qkv_g = qkv.cuda()
        sl = lambda t, a, n: t[:, a * d:(a + n) * d].view(t.shape[0], n, d)
        q, k, v = sl(qkv, 0, hq), sl(qkv, hq, hk), sl(qkv, hq + hk, hk)
        qg, kg, vg = sl(qkv_g, 0, hq), sl(qkv_g, hq, hk), sl(qkv_g, hq + hk, hk)
    else:
        q, k, v = randn((tq, hq, d), dtype, seed), randn((tk, hk, d), dtype, seed + 1), randn((tk, hk, d), dtype, seed + 2)
        qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    do = randn((tq, hq, d), dtype, seed + 3)
    mq, mk = max(lens_q), max(lens_k)
    res = _Clib.pymha_varlen_fwd(qg, kg, vg, cq.cuda(), ck.cuda(), mq, mk, 0.0, scale, causal, False, 0, False)
    assert len(res) == 8
    out, lse = res[0], res[5]
    assert res[4] is out and res[1] is qg
    oo, lo = OA.attn_fwd(q, k, v, cq, ck, scale, causal, oracle_dtype)
    assert_close(out, oo, dtype, "out")
    for i, n in enumerate(lens_q):
        if n:
            assert_close(lse[i, :, :n], lo[i, :, :n], torch.float32, f"lse[{i}]")
    # backward consumes the forward's own (rounded) out and lse, like the layer does
    stream = torch.cuda.current_stream()
    r = _Clib.pymha_varlen_bwd(do.cuda(), qg, kg, vg, out, lse, cq.cuda(), ck.cuda(), mq, mk, 0.0, scale, causal,
                               None, False, 0, False, stream.cuda_stream)
    assert len(r) == 4
    dq, dk, dv, dl = r
    lse_cpu = lse.cpu().double()
    dqo, dko, dvo, dlo = OA.attn_bwd(do, q, k, v, out.cpu(), lse_cpu, cq, ck, scale, causal, oracle_dtype)
    assert_close(dq, dqo, dtype, "dq")
    assert_close(dk, dko, dtype, "dk")
    assert_close(dv, dvo, dtype, "dv")
    for i, n in enumerate(lens_q):
        if n:
            assert_close(dl[i, :, :n], dlo[i, :, :n], torch.float32, f"delta[{i}]")
    return out, lse, dq, dk, dv


@pytest.fixture(params=[True, False], ids=["keep_ds", "recompute"])
def ds_path(request):
    """Head dim 128 has two backward paths: dQ from the dS that the dK/dV pass keeps, or from recomputed S and dP."""
    from dhellam_amd import _Clib
    _Clib.set_attn_bwd_ds_limit(_Clib.ATTN_BWD_DS_LIMIT_DEFAULT if request.param else 0)
    yield request.param
    _Clib.set_attn_bwd_ds_limit()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lens_q,lens_k,hq,hk,d,causal", [
    ([1024], [1024], 8, 1, 128, True),          # the 70B shard's head layout, shortened
    ([512, 512], [512, 512], 16, 16, 64, True),  # MHA, d 64, two sequences
    ([100, 257, 64, 1], [100, 257, 64, 1], 4, 2, 128, True),   # ragged
    ([300], [200], 4, 2, 128, False),            # rectangular, non-causal
    ([128, 77], [640, 33], 6, 3, 64, False),
    ([2048], [1024], 8, 2, 128, False),          # ring 'lower' shape
    ([1024], [2048], 8, 2, 128, False),          # ring 'upper' shape
    ([384, 129], [384, 129], 4, 4, 128, True),   # MHA at d 128: dK/dV written directly (no head split)
    ([128] * 4, [512] * 4, 64, 16, 128, False),  # many kv heads: two query heads per dK/dV workgroup
    ([0, 65, 33], [0, 65, 33], 4, 2, 128, True),   # an empty sequence in the batch
])
def test_attention_16bit(dtype, lens_q, lens_k, hq, hk, d, causal, ds_path):
    if d != 128 and not ds_path:
        pytest.skip("one backward path at this head dim")
    _run_fwd_bwd(dtype, lens_q, lens_k, hq, hk, d, causal)


@pytest.mark.parametrize("lens_q,lens_k,hq,hk,causal", [
    ([1024], [1024], 8, 1, True), ([100, 257, 64, 1], [100, 257, 64, 1], 4, 2, True), ([300, 40], [200, 97], 4, 2, False),
    ([2048], [1000], 8, 2, False),
])
def test_attention_backward_paths_agree(lens_q, lens_k, hq, hk, causal):
    """The two backward paths at head dim 128 on the same inputs: dV comes from the same kernel arithmetic
    (bit-identical); dK and dQ use delta = rowsum(dO * O), which the two paths sum in a different order (the delta
    kernel / the prologue of the recomputing dQ kernel), so a few of their elements differ in the last place."""
    from dhellam_amd import _Clib
    dtype, d = torch.bfloat16, 128
    cq, ck = _cu(lens_q).cuda(), _cu(lens_k).cuda()
    tq, tk, mq, mk = sum(lens_q), sum(lens_k), max(lens_q), max(lens_k)
    scale = 1.0 / math.sqrt(d)
    q, k, v, do = (randn((t, h, d), dtype, 30 + i).cuda() for i, (t, h) in enumerate(((tq, hq), (tk, hk), (tk, hk), (tq, hq))))
    res = _Clib.pymha_varlen_fwd(q, k, v, cq, ck, mq, mk, 0.0, scale, causal, False, 0, False)
    out, lse = res[0], res[5]
    sp = torch.cuda.current_stream().cuda_stream
    got = []
    try:
        for limit in (_Clib.ATTN_BWD_DS_LIMIT_DEFAULT, 0):
            _Clib.set_attn_bwd_ds_limit(limit)
            dq, dk, dv = torch.full_like(q, float("nan")), torch.full_like(k, float("nan")), torch.full_like(v, float("nan"))
            _Clib._attn_bwd_raw(do, q, k, v, out, lse, dq, dk, dv, None, cq, ck, mq, mk, scale, causal, sp)
            got.append((dq, dk, dv))
    finally:
        _Clib.set_attn_bwd_ds_limit()
    assert torch.equal(got[0][2], got[1][2])
    assert_close(got[0][1], got[1][1].double().cpu(), dtype, "dk of the two paths", scale=0.25)
    assert_close(got[0][0], got[1][0].double().cpu(), dtype, "dq of the two paths", scale=0.25)


def test_attention_packed_qkv_views():
    _run_fwd_bwd(torch.bfloat16, [384, 128], [384, 128], 8, 1, 128, True, packed=True)


def test_attention_full_70b_shard_shape():
    # 8 q heads + 1 kv head, d 128, 4096 tokens, causal, bf16; oracle in fp32 to keep the CPU time in seconds
    _run_fwd_bwd(torch.bfloat16, [4096], [4096], 8, 1, 128, True, oracle_dtype=torch.float32)


@pytest.mark.parametrize("lens_q,lens_k,hq,hk,d,causal", [
    ([512, 512], [512, 512], 16, 16, 64, True),  # the fp32 parity configuration
    ([130, 7], [130, 7], 4, 2, 32, True),
    ([50], [200], 2, 1, 256, False),
    ([70], [70], 3, 3, 20, True),
])
def test_attention_fp32(lens_q, lens_k, hq, hk, d, causal):
    _run_fwd_bwd(torch.float32, lens_q, lens_k, hq, hk, d, causal)


@pytest.mark.parametrize("dtype,hq,hk,d", [(torch.bfloat16, 4, 2, 128), (torch.float16, 32, 8, 128), (torch.bfloat16, 2, 2, 64),
                                         (torch.float32, 2, 1, 32)])
def test_attention_backward_accumulates_dq(dtype, hq, hk, d, ds_path):
    """dh_attn_bwd_acc with accumulate_dq: dq += the call's gradient (one rounding of the fp32 sum); dk, dv and a
    call without the flag are those of dh_attn_bwd."""
    from dhellam_amd import _Clib
    lens = [200, 56] if hq < 32 else [640]
    cu = _cu(lens).cuda()
    t, m, scale = sum(lens), max(lens), 1.0 / math.sqrt(d)
    q, k, v, do = (randn((t, h, d), dtype, 10 + i).cuda() for i, h in enumerate((hq, hk, hk, hq)))
    res = _Clib.pymha_varlen_fwd(q, k, v, cu, cu, m, m, 0.0, scale, True, False, 0, False)
    out, lse = res[0], res[5]
    sp = torch.cuda.current_stream().cuda_stream
    dq0, dk0, dv0 = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    _Clib._attn_bwd_raw(do, q, k, v, out, lse, dq0, dk0, dv0, None, cu, cu, m, m, scale, True, sp)
    base = randn((t, hq, d), dtype, 20).cuda()
    dq1, dk1, dv1 = base.clone(), torch.empty_like(k), torch.empty_like(v)
    _Clib._attn_bwd_raw(do, q, k, v, out, lse, dq1, dk1, dv1, None, cu, cu, m, m, scale, True, sp, accumulate_dq=True)
    assert torch.equal(dk1, dk0) and torch.equal(dv1, dv0)
    # the kernel adds its fp32 gradient before rounding, so it is at least as close to the exact sum as adding the
    # rounded gradient: compare with base + dq0 at the operator tolerance, and bit for bit where nothing was there
    assert_close(dq1, base.double().cpu() + dq0.double().cpu(), dtype, "dq accumulated")
    dq2 = torch.zeros_like(q)
    _Clib._attn_bwd_raw(do, q, k, v, out, lse, dq2, dk1, dv1, None, cu, cu, m, m, scale, True, sp, accumulate_dq=True)
    assert torch.equal(dq2, dq0)


def test_attention_is_deterministic():
    a = _run_fwd_bwd(torch.bfloat16, [700], [700], 8, 2, 128, True)
    b = _run_fwd_bwd(torch.bfloat16, [700], [700], 8, 2, 128, True)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_attention_profiling_and_errors():
    from dhellam_amd import _Clib
    q = randn((256, 4, 128), torch.bfloat16, 0).cuda()
    cu = _cu([256]).cuda()
    res = _Clib.pymha_varlen_fwd(q, q, q, cu, cu, 256, 256, 0.0, 0.1, True, False, 0, True)
    assert len(res) == 9 and res[8].device.type == "cpu" and res[8].item() > 0
    with pytest.raises(RuntimeError):
        _Clib.pymha_varlen_fwd(q, q, q, cu, cu, 256, 256, 0.1, 0.1, True, False, 0, False)   # dropout
    # the C ABI itself takes the compiled head dims only (the bindings pad other sizes before they call it)
    from dhellam_amd import _lib
    q72 = randn((256, 4, 72), torch.bfloat16, 0).cuda()
    o72, l72 = torch.empty_like(q72), torch.empty(1, 4, 256, device="cuda")
    rc = _lib.load().dh_attn_fwd(q72.data_ptr(), q72.data_ptr(), q72.data_ptr(), o72.data_ptr(), l72.data_ptr(),
                                 cu.data_ptr(), cu.data_ptr(), 1, 256, 256, 4, 4, 72, 288, 288, 288, 288, 0.1, 1,
                                 _lib.DH_BF16, torch.cuda.current_stream().cuda_stream)
    assert rc == -1 and "head dim" in _lib.load().dh_last_error().decode()
    k3 = randn((256, 3, 128), torch.bfloat16, 0).cuda()
    with pytest.raises(RuntimeError, match="multiple"):
        _Clib.pymha_varlen_fwd(q, k3, k3, cu, cu, 256, 256, 0.0, 0.1, True, False, 0, False)


# ------------------------------------------------------------------------------------------
# merge and ring step
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_merge_kernel(dtype):
    from dhellam_amd import _Clib
    b, sq, hq, d = 2, 96, 3, 64
    row_begin, rows = [0, 0, 48, 48], [96, 96, 48, 48]
    outs = [randn((b * n, hq, d), dtype, 10 + i) for i, n in enumerate(rows)]
    lses = [randn((b, hq, n), torch.float32, 20 + i, std=3.0) for i, n in enumerate(rows)]
    out = torch.empty((b * sq, hq, d), dtype=dtype, device="cuda")
    lse = torch.empty((b, hq, sq), dtype=torch.float32, device="cuda")
    _Clib.pyattn_merge([o.cuda() for o in outs], [l.cuda() for l in lses], row_begin, rows, out, lse)
    oo, lo = OA.merge(outs, lses, row_begin, rows, b, sq, hq, d)
    assert_close(out, oo, dtype, "merged out")
    assert_close(lse, lo, torch.float32, "merged lse")


def _ring_inputs(dtype, b, c, hq, hk, d, cp, seed=0):
    q = randn((b, 2, c, hq, d), dtype, seed)
    chunks = [(randn((b, 2, c, hk, d), dtype, seed + 10 + 2 * i), randn((b, 2, c, hk, d), dtype, seed + 11 + 2 * i))
              for i in range(cp)]
    dout = randn((b, 2, c, hq, d), dtype, seed + 99)
    return q, chunks, dout


def _ring_gpu(q, chunks, dout, rank, cp):
    from dhellam_amd.operators.ring_attn import RingGroup, fa_cp_block_bwd, fa_cp_block_fwd
    b, _, c = q.shape[:3]
    s = 2 * c
    grp = RingGroup(rank, cp)
    cu = torch.arange(0, (b + 1) * s, s, dtype=torch.int32).cuda()
    bufs = [torch.stack((k, v)).cuda() for k, v in chunks]
    qg = q.cuda()
    carry = [qg, bufs, None, None, None, None, None, 0]
    for i in range(cp):
        r = fa_cp_block_fwd(carry[0], cu, cu, s, s, carry[1], carry[2], carry[3], carry[4], carry[5], carry[6], i,
                            True, grp, list(range(cp)), None)
        if i < cp - 1:
            carry, reqs = r
            assert reqs == [] and carry[-1] == i + 1
        else:
            out, q_ret, kv_ret, lse, rng = r
    assert q_ret is qg and kv_ret is bufs[-1]
    state = [dout.cuda(), None, None, bufs, 0]
    for i in range(cp + 1):
        r = fa_cp_block_bwd(state[0], out, qg, state[1], None, state[2], lse, rng, cu, cu, s, s, state[3], i, True,
                            grp, list(range(cp)), None)
        if i < cp:
            state, reqs = r
        else:
            dq, dkv = r
    return out, lse, dq, dkv


@pytest.mark.parametrize("dtype,b,c,hq,hk,d", [(torch.bfloat16, 1, 128, 4, 2, 128), (torch.bfloat16, 1, 96, 2, 2, 64),
                                                 (torch.float32, 1, 48, 2, 1, 32), (torch.bfloat16, 2, 64, 4, 2, 128)])
@pytest.mark.parametrize("rank", [0, 1, 3])
def test_ring_step_matches_oracle_and_dense(dtype, b, c, hq, hk, d, rank):
    cp = 4
    q, chunks, dout = _ring_inputs(dtype, b, c, hq, hk, d, cp)
    scale = 1.0 / math.sqrt(d)
    out, lse, dq, dkv = _ring_gpu(q, chunks, dout, rank, cp)
    oo, lo, _ = OA.ring_fwd(q, chunks, rank, scale)
    assert_close(out, oo, dtype, "ring out")
    assert_close(lse, lo, torch.float32, "ring lse")
    # the same thing as ONE dense causal attention over the zig-zag order
    do_, lo_ = OA.zigzag_dense(q, chunks, rank, scale)
    assert_close(out.view(b, 2 * c, hq, d), do_, dtype, "ring out vs dense")
    # backward: oracle ring with the GPU's own merged out/lse
    dqo, dkvo = OA.ring_bwd(dout, out.cpu(), lse.cpu().double(), q, chunks, rank, scale)
    assert_close(dq.view(q.shape), dqo, dtype, "ring dq")
    for s in range(cp):
        assert_close(dkv[s][0], dkvo[s][0], dtype, f"ring dk[{s}]")
        assert_close(dkv[s][1], dkvo[s][1], dtype, f"ring dv[{s}]")


@pytest.mark.parametrize("rank", [0, 1, 3])
def test_ring_step_full_size(rank):
    """The ring configuration at its full shape (q [1, 2, 2048, 32, 128], four visiting KV chunks of 8 kv heads;
    rank 0: a diagonal step and three half-q steps, rank 3: a diagonal step and three half-kv steps, rank 1:
    both kinds): forward and backward against ONE dense attention over the zig-zag positions, evaluated by the
    oracle in fp32 with its matmuls on the GPU (the [32, 4096, 16384] score tensor is 8.6 GB), gradients by
    autograd.  16-bit tolerance."""
    dtype, b, c, hq, hk, d, cp = torch.bfloat16, 1, 2048, 32, 8, 128, 4
    q, chunks, dout = _ring_inputs(dtype, b, c, hq, hk, d, cp, seed=3)
    scale = 1.0 / math.sqrt(d)
    out, lse, dq, dkv = _ring_gpu(q, chunks, dout, rank, cp)
    qr = q.cuda().float().requires_grad_()
    cr = [(k.cuda().float().requires_grad_(), v.cuda().float().requires_grad_()) for k, v in chunks]
    do_, lo_ = OA.zigzag_dense(qr, cr, rank, scale, dtype=torch.float32)
    assert_close(out.view(b, 2 * c, hq, d), do_, dtype, "ring out vs dense")
    assert_close(lse, lo_, torch.float32, "ring lse")
    (do_ * dout.cuda().float().view(b, 2 * c, hq, d)).sum().backward()
    assert_close(dq.view(q.shape), qr.grad, dtype, "ring dq")
    for s in range(cp):
        assert_close(dkv[s][0], cr[s][0].grad, dtype, f"ring dk[{s}]")
        assert_close(dkv[s][1], cr[s][1].grad, dtype, f"ring dv[{s}]")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d,lens,hq,hk,causal", [
    (96, [160, 37], 4, 2, True),            # compiled head dims beside 64 / 128 ...
    (192, [130, 64], 4, 1, True),
    (256, [96, 71], 2, 2, True),
    (256, [200], 4, 2, False),
    (80, [150, 33], 4, 2, True),            # ... and sizes that run zero-padded to the next one (the reference takes
    (40, [129], 2, 2, False),               # any d <= 256 and pads to a multiple of 8, flash_atten.cu:284,303-312)
    (160, [100, 90], 2, 1, True),
])
def test_attention_other_head_dims(dtype, d, lens, hq, hk, causal):
    """16-bit attention for head dims other than 64 / 128, forward and backward against the fp64 oracle, through
    the Python mirror of the binding and through the compiled extension (same bits)."""
    from dhellam_amd import _Clib
    import dhellam._Clib as C
    cu = _cu(lens)
    t, m = int(cu[-1]), max(lens)
    scale = 1.0 / math.sqrt(d)
    q, k, v, do = (randn((t, h, d), dtype, s) for s, h in ((0, hq), (1, hk), (2, hk), (3, hq)))
    qg, kg, vg, cug = q.cuda(), k.cuda(), v.cuda(), cu.cuda()
    res = _Clib.pymha_varlen_fwd(qg, kg, vg, cug, cug, m, m, 0.0, scale, causal, False, 0, False)
    out, lse = res[0], res[5]
    assert out.shape == q.shape
    d_run = res[4].shape[-1]
    assert d_run in _Clib.HEAD_DIMS_16BIT and d_run >= d and res[1].shape[-1] == d_run      # the "padded" slots
    oo, lo = OA.attn_fwd(q, k, v, cu, cu, scale, causal, torch.float64)
    assert_close(out, oo, dtype, "out")
    for i, n in enumerate(lens):
        assert_close(lse[i, :, :n], lo[i, :, :n], torch.float32, f"lse[{i}]")
    if d_run != d:
        assert torch.count_nonzero(res[4][..., d:]) == 0                                    # padding columns stay zero
    outc = out.contiguous()
    sp = torch.cuda.current_stream().cuda_stream
    dq, dk, dv, _ = _Clib.pymha_varlen_bwd(do.cuda(), qg, kg, vg, outc, lse, cug, cug, m, m, 0.0, scale, causal, None,
                                           False, 0, False, sp)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    dqo, dko, dvo, _ = OA.attn_bwd(do, q, k, v, outc.cpu(), lse.cpu().double(), cu, cu, scale, causal, torch.float64)
    assert_close(dq, dqo, dtype, "dq")
    assert_close(dk, dko, dtype, "dk")
    assert_close(dv, dvo, dtype, "dv")
    # the compiled extension pads and runs the same kernels
    rc = C.pymha_varlen_fwd(qg, kg, vg, cug, cug, m, m, 0.0, scale, causal, False, 0, False)
    assert torch.equal(rc[0], out) and rc[4].shape[-1] == d_run
    assert all(torch.equal(rc[5][i, :, :n], lse[i, :, :n]) for i, n in enumerate(lens))   # (entries past a sequence are not written)
    gc = C.pymha_varlen_bwd(do.cuda(), qg, kg, vg, outc, lse, cug, cug, m, m, 0.0, scale, causal, None, False, 0, False, sp)
    torch.cuda.synchronize()
    for a, b_ in zip(gc[:3], (dq, dk, dv)):
        assert torch.equal(a, b_)


def test_attention_head_dim_above_256_is_refused():
    from dhellam_amd import _Clib
    q = torch.zeros(8, 1, 264, dtype=torch.bfloat16, device="cuda")
    cu = _cu([8]).cuda()
    with pytest.raises(RuntimeError, match="256"):
        _Clib.pymha_varlen_fwd(q, q, q, cu, cu, 8, 8, 0.0, 1.0, True, False, 0, False)
