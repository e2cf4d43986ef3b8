"""The compiled pybind11 extension ``dhellam._Clib`` (the reference builds a module of that name from
csrc/torchapi.cpp:2-9) on the GPU: attention forward + backward and ``pygemm`` through it against the oracle, the
return conventions of csrc/operators/flash_atten.cu:429-433,752-756 (list lengths, the extra CPU tensor of
milliseconds when profiling), the raw ``stream_ptr`` of the backward (ops.h:52) and a non-zero ``math_sm_count``.
Tolerances: rel-err <= 1e-2 (bf16), <= 1e-5 (fp32)."""
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


@pytest.mark.parametrize("dtype,lens,hq,hk,d,causal", [
    (torch.bfloat16, [192, 77], 8, 2, 128, True),
    (torch.bfloat16, [130], 4, 4, 64, False),
    (torch.float32, [96, 40], 4, 2, 64, True),
])
def test_attention_through_the_compiled_extension(dtype, lens, hq, hk, d, causal):
    import dhellam._Clib as C
    assert C.__file__.endswith(".so")
    cu = _cu(lens)
    t, m = int(cu[-1]), max(lens)
    scale = 1.0 / math.sqrt(d)
    q, k, v, do = (randn((t, h, d), dtype, s) for s, h in ((0, hq), (1, hk), (2, hk), (3, hq)))
    qg, kg, vg, cug = q.cuda(), k.cuda(), v.cuda(), cu.cuda()
    res = C.pymha_varlen_fwd(qg, kg, vg, cug, cug, m, m, 0.0, scale, causal, False, 0, False)
    assert len(res) == 8 and res[7].dtype == torch.int64 and res[7].numel() == 2 and res[6].numel() == 0
    out, lse = res[0], res[5]
    assert res[4].data_ptr() == out.data_ptr() and res[1].data_ptr() == qg.data_ptr()
    oo, lo = OA.attn_fwd(q, k, v, cu, cu, scale, causal, torch.float64)
    assert_close(out, oo, dtype, "out")
    for i, n in enumerate(lens):
        assert_close(lse[i, :, :n], lo[i, :, :n], torch.float32, f"lse[{i}]")
    # the backward on a raw stream handle that is not torch's current stream
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    r = C.pymha_varlen_bwd(do.cuda(), qg, kg, vg, out, lse, cug, cug, m, m, 0.0, scale, causal, None, False, 0, False,
                           side.cuda_stream)
    assert len(r) == 4
    side.synchronize()
    dq, dk, dv, delta = r
    dqo, dko, dvo, dlo = OA.attn_bwd(do, q, k, v, out.cpu(), lse.cpu().double(), cu, cu, scale, causal, torch.float64)
    assert_close(dq, dqo, dtype, "dq")
    assert_close(dk, dko, dtype, "dk")
    assert_close(dv, dvo, dtype, "dv")
    for i, n in enumerate(lens):
        assert_close(delta[i, :, :n], dlo[i, :, :n], torch.float32, f"delta[{i}]")
        assert torch.count_nonzero(delta[i, :, n:]) == 0          # rows past the sequence stay zero
    # same numbers as the ctypes mirror of the module, bit for bit
    from dhellam_amd import _Clib as P
    r2 = P.pymha_varlen_bwd(do.cuda(), qg, kg, vg, out, lse, cug, cug, m, m, 0.0, scale, causal, None, False, 0, False,
                            torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for a, b in zip(r[:3], r2[:3]):
        assert torch.equal(a, b)


def test_profiling_and_confinement_through_the_compiled_extension():
    import dhellam._Clib as C
    dtype, hq, hk, d, n = torch.bfloat16, 4, 1, 128, 256
    cu = _cu([n]).cuda()
    q, k, v = randn((n, hq, d), dtype, 0).cuda(), randn((n, hk, d), dtype, 1).cuda(), randn((n, hk, d), dtype, 2).cuda()
    plain = C.pymha_varlen_fwd(q, k, v, cu, cu, n, n, 0.0, 0.1, True, False, 0, False)
    timed = C.pymha_varlen_fwd(q, k, v, cu, cu, n, n, 0.0, 0.1, True, False, 0, True)
    assert len(timed) == 9 and not timed[8].is_cuda and timed[8].dtype == torch.float32 and float(timed[8]) > 0
    masked = C.pymha_varlen_fwd(q, k, v, cu, cu, n, n, 0.0, 0.1, True, False, 16, False)     # on 16 compute units
    torch.cuda.synchronize()
    assert torch.equal(plain[0], timed[0]) and torch.equal(plain[0], masked[0]) and torch.equal(plain[5], masked[5])
    do = randn((n, hq, d), dtype, 3).cuda()
    r = C.pymha_varlen_bwd(do, q, k, v, plain[0], plain[5], cu, cu, n, n, 0.0, 0.1, True, None, True, -16, True, 0)
    assert len(r) == 5 and float(r[4]) > 0
    with pytest.raises(RuntimeError, match="math_sm_count"):
        C.pymha_varlen_fwd(q, k, v, cu, cu, n, n, 0.0, 0.1, True, False, 100000, False)


@pytest.mark.parametrize("layout", ["TN", "NN", "NT"])
def test_pygemm_through_the_compiled_extension(layout):
    """csrc/operators/gemm.cu:3-170: D = op(B) @ op(A) over row-major tensors."""
    import dhellam._Clib as C
    dtype, t, n, k = torch.bfloat16, 256, 384, 512
    x, w, dy = randn((t, k), dtype, 0), randn((n, k), dtype, 1, 0.05), randn((t, n), dtype, 2)
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    if layout == "TN":        # forward: x @ w^T
        a, b, ref = w, x, x.double() @ w.double().t()
    elif layout == "NN":      # data gradient: dy @ w
        a, b, ref = w, dy, dy.double() @ w.double()
    else:                     # weight gradient: dy^T @ x
        a, b, ref = x, dy, dy.double().t() @ x.double()
    out = torch.empty(ref.shape, dtype=dtype, device="cuda")
    ms = C.pygemm(a.cuda(), b.cuda(), out, ws, ws.numel(), layout[0] == "T", layout[1] == "T", False, 0, False)
    assert ms == 0.0
    assert_close(out, ref, dtype, layout)
    # accumulate on top, timed
    ms = C.pygemm(a.cuda(), b.cuda(), out, ws, ws.numel(), layout[0] == "T", layout[1] == "T", True, 0, True)
    assert ms > 0.0
    assert_close(out, 2 * ref, dtype, layout + " accumulated")


def test_elementwise_names_through_the_compiled_extension():
    import dhellam._Clib as C
    x, bias, res = (randn((64, 256), torch.float16, s).cuda() for s in range(3))
    out = torch.empty_like(x)
    assert C.pygelu(x, out, False) == 0.0
    ref = torch.nn.functional.gelu(x.double().cpu(), approximate="tanh")
    assert_close(out, ref, torch.float16, "gelu")
    assert C.pybda(x, bias, res, out, 0.0, True) > 0.0
    assert_close(out, (x.double() + bias.double() + res.double()).cpu(), torch.float16, "bda")
    assert torch.equal(C.add_tensors(x, bias), x + bias)
    with pytest.raises(RuntimeError, match="prob"):
        C.pybda(x, bias, res, out, 0.1, False)


# ---- what the C ABI checks instead of trusting the caller -----------------------------------------------------------
def test_attention_backward_checks_its_workspace_size():
    """``dh_attn_bwd`` is told how large its workspace is: less than the minimum is refused before anything is
    launched, and whether dS is kept follows what fits the given size, not a process-wide setting read at another
    moment (raising the limit after the workspace was sized must not make the call write past it)."""
    from dhellam_amd import _Clib, _lib
    lib = _lib.load()
    dtype, hq, hk, d, n = torch.bfloat16, 8, 1, 128, 512
    cu = _cu([n]).cuda()
    q, k, v, do = (randn((n, h, d), dtype, s).cuda() for s, h in ((0, hq), (1, hk), (2, hk), (3, hq)))
    out, lse = _Clib.pymha_varlen_fwd(q, k, v, cu, cu, n, n, 0.0, 0.1, True, False, 0, False)[0::5]
    args = (q.shape[0], k.shape[0], 1, n, hq, hk, d, _lib.DH_BF16)
    _Clib.set_attn_bwd_ds_limit(0)
    try:
        small = lib.dh_attn_bwd_workspace_bytes(*args)              # sized while dS is never kept
        assert small == lib.dh_attn_bwd_min_workspace_bytes(*args)
    finally:
        _Clib.set_attn_bwd_ds_limit()
    full = lib.dh_attn_bwd_workspace_bytes(*args)
    assert full > small                                             # this shape would keep dS
    guard = 1 << 20
    buf = torch.full((full + guard,), 0x5A, dtype=torch.uint8, device="cuda")

    def run(nbytes):
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        rc = lib.dh_attn_bwd(do.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                             dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), None, buf.data_ptr(), nbytes,
                             cu.data_ptr(), cu.data_ptr(), 1, n, n, n, n, hq, hk, d, hq * d, hk * d, hk * d, hq * d,
                             hq * d, hq * d, hk * d, hk * d, 0.1, 1, _lib.DH_BF16, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return rc, dq, dk, dv

    rc, *_ = run(small - 256)
    assert rc == -1 and "smaller" in lib.dh_last_error().decode()
    # the limit is back at its default (it would keep dS), the workspace is the small one: nothing behind it is touched
    buf.fill_(0x5A)
    rc, dq_a, dk_a, dv_a = run(small)
    assert rc == 0
    assert bool((buf[small:] == 0x5A).all()), "the backward wrote past the workspace it was given"
    rc, dq_b, dk_b, dv_b = run(full)
    assert rc == 0
    assert bool((buf[full:] == 0x5A).all())
    assert not bool((buf[small:full] == 0x5A).all())                # ... and with room for it dS was kept
    dqo, dko, dvo, _ = OA.attn_bwd(do.cpu(), q.cpu(), k.cpu(), v.cpu(), out.cpu(), lse.cpu().double(), cu.cpu(), cu.cpu(), 0.1, True,
                                   torch.float64)
    for got, ref, what in ((dq_a, dqo, "dq"), (dk_a, dko, "dk"), (dv_a, dvo, "dv"), (dq_b, dqo, "dq kept"),
                           (dk_b, dko, "dk kept"), (dv_b, dvo, "dv kept")):
        assert_close(got, ref, dtype, what)


def test_norm_backward_and_sort_check_their_workspace_size():
    from dhellam_amd import _lib
    lib = _lib.load()
    rows, cols = 64, 1024
    x, dy, g = (torch.randn(rows, cols, device="cuda") for _ in range(3))
    rs = torch.rand(rows, device="cuda") + 0.5
    dx, dg = torch.empty_like(x), torch.empty(cols, device="cuda")
    need = lib.dh_norm_bwd_workspace_bytes(rows, cols)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    call = lambda nbytes: lib.dh_norm_bwd(dy.data_ptr(), x.data_ptr(), None, rs.data_ptr(), g[0].data_ptr(), None,
                                          dx.data_ptr(), dg.data_ptr(), None, ws.data_ptr(), nbytes, rows, cols, 0, 0,
                                          _lib.DH_F32, st)
    assert call(need - 1) == -1 and "smaller" in lib.dh_last_error().decode()
    assert call(need) == 0
    n, e = 4096, 8
    idx = torch.randint(0, e, (n,), dtype=torch.int32, device="cuda")
    tpe, offs = torch.empty(e, dtype=torch.int32, device="cuda"), torch.empty(e + 1, dtype=torch.int32, device="cuda")
    sidx, dest = torch.empty(n, dtype=torch.int32, device="cuda"), torch.empty(n, dtype=torch.int32, device="cuda")
    need = lib.dh_moe_sort_workspace_bytes(n, e)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    call = lambda nbytes: lib.dh_moe_sort(idx.data_ptr(), tpe.data_ptr(), offs.data_ptr(), sidx.data_ptr(),
                                          dest.data_ptr(), ws.data_ptr(), nbytes, n, e, st)
    assert call(need - 1) == -1 and "smaller" in lib.dh_last_error().decode()
    assert call(need) == 0
    torch.cuda.synchronize()
    assert int(tpe.sum()) == n
