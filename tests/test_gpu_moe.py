"""GPU parity of MoE routing / sort / permute / unpermute (bit-exact indices) and of the
MFMA grouped GEMM and expert FFN against the oracle."""
import numpy as np
import pytest
import torch

from oracle import moe as OM
from tests.util import assert_close, randn, rel_err

# Bound on the distance between the 16-bit expert FFN and the oracle that keeps h and a exact: two 16-bit stores
# on the way forward and two gradients stored on the way back, each off by up to 2^-9 of itself.
UNROUNDED_BOUND = 1e-2      # measured: 3.4e-3 .. 3.5e-3

pytestmark = pytest.mark.gpu


def _logits(T, E, seed, ties=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, E), generator=g, dtype=torch.float32)
    if ties:
        x = torch.round(x * 2) / 2          # many exact ties
    return x


@pytest.mark.parametrize("T,E,k,ties", [(8192, 8, 2, False), (1000, 8, 2, True), (33, 64, 8, True), (5, 3, 1, False),
                                         (4096, 16, 4, True)])
def test_route_topk_bit_exact(T, E, k, ties):
    from dhellam_amd.operators.moe import route_topk
    lg = _logits(T, E, 1, ties)
    idx, gates, ms = route_topk(lg.cuda(), k)
    io, go = OM.route_topk(lg.numpy(), k)
    assert np.array_equal(idx.cpu().numpy(), io), "top-k indices must be bit-exact"
    assert_close(gates, torch.from_numpy(go), torch.float32, "gates")
    assert torch.allclose(gates.sum(1).cpu(), torch.ones(T), atol=1e-6)


@pytest.mark.parametrize("T,E,k", [(8192, 8, 2), (1000, 8, 2), (3000, 64, 8), (1, 4, 1), (1025, 5, 3)])
def test_sort_bit_exact(T, E, k):
    from dhellam_amd.operators.moe import sort_assignments
    io, _ = OM.route_topk(_logits(T, E, 2, True).numpy(), k)
    plan, _ = sort_assignments(torch.from_numpy(io).cuda(), E)
    tpe, offs, sidx, dest = OM.sort_assignments(io, E)
    assert np.array_equal(plan.tokens_per_expert.cpu().numpy(), tpe)
    assert np.array_equal(plan.expert_offsets.cpu().numpy(), offs)
    assert np.array_equal(plan.sorted_idx.cpu().numpy(), sidx), "stable sort order must be bit-exact"
    assert np.array_equal(plan.dest_row.cpu().numpy(), dest)


def test_sort_skewed_and_empty_experts():
    from dhellam_amd.operators.moe import sort_assignments
    idx = np.zeros((5000, 2), dtype=np.int32)
    idx[:, 1] = 7                                  # experts 1..6 receive nothing
    plan, _ = sort_assignments(torch.from_numpy(idx).cuda(), 8)
    tpe, offs, sidx, dest = OM.sort_assignments(idx, 8)
    assert np.array_equal(plan.tokens_per_expert.cpu().numpy(), tpe)
    assert np.array_equal(plan.sorted_idx.cpu().numpy(), sidx)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,H,E,k,e_lo,e_hi", [(8192, 4096, 8, 2, 0, 2), (777, 520, 8, 2, 2, 5), (300, 100, 4, 1, 0, 4),
                                                (64, 256, 8, 2, 7, 8)])
def test_permute_unpermute(dtype, T, H, E, k, e_lo, e_hi):
    from dhellam_amd.operators import moe
    lg = _logits(T, E, 3)
    idx, gates, _ = moe.route_topk(lg.cuda(), k)
    plan, _ = moe.sort_assignments(idx, E)
    io, go = OM.route_topk(lg.numpy(), k)
    tpe, offs, sidx, dest = OM.sort_assignments(io, E)
    R = int(offs[e_hi] - offs[e_lo])
    max_rows = R + 37
    x = randn((T, H), dtype, 4)
    xp, _ = moe.permute_fwd(x.cuda(), plan, e_lo, e_hi, max_rows)
    xo = OM.permute(x, sidx, offs, e_lo, e_hi, k)
    assert torch.equal(xp[:R].cpu(), xo.to(dtype)), "permute is a pure row copy: must be bit-exact"
    assert xp[R:].abs().max().item() == 0 if max_rows > R else True
    # unpermute with gates
    y = randn((max_rows, H), dtype, 5)
    out, _ = moe.unpermute_fwd(y.cuda(), plan, gates, e_lo, e_hi)
    oo = OM.unpermute(y[:R], dest, offs, e_lo, e_hi, T, k, gates.cpu())
    assert_close(out, oo, dtype, "unpermute")
    # backward pieces
    dxo = OM.unpermute(y[:R], dest, offs, e_lo, e_hi, T, k, None)
    dx, _ = moe.permute_bwd(y.cuda(), plan, e_lo, e_hi)
    assert_close(dx, dxo, dtype, "permute_bwd")
    dout = randn((T, H), dtype, 6)
    dy, dg, _ = moe.unpermute_bwd(dout.cuda(), y.cuda(), plan, gates, e_lo, e_hi, max_rows)
    dyo = OM.permute(dout, sidx, offs, e_lo, e_hi, k, row_scale=gates.cpu())
    assert_close(dy[:R], dyo, dtype, "unpermute_bwd dy")
    dgo = OM.gate_grad(dout, y[:R], dest, offs, e_lo, e_hi, T, k)
    assert_close(dg, dgo, torch.float32, "dgates")


def test_permute_roundtrip_identity():
    """top-1, gates 1, all experts local: unpermute(permute(x)) == x exactly."""
    from dhellam_amd.operators import moe
    T, H, E = 2048, 512, 8
    lg = _logits(T, E, 7)
    idx, gates, _ = moe.route_topk(lg.cuda(), 1)
    plan, _ = moe.sort_assignments(idx, E)
    x = randn((T, H), torch.bfloat16, 8).cuda()
    xp, _ = moe.permute_fwd(x, plan, 0, E, T)
    back, _ = moe.unpermute_fwd(xp, plan, torch.ones_like(gates), 0, E)
    assert torch.equal(back, x)
    assert int(plan.tokens_per_expert.sum()) == T


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,N,K", [([300, 212], 512, 256), ([1000, 0, 24], 1024, 520), ([2048, 2048], 2048, 1024),
                                       ([5], 64, 64),
                                       # enough 256x256 tiles for the direct global->LDS kernels (NT and NN), with an
                                       # empty group, a 37-row group and three k slices
                                       ([2100, 0, 1990, 37], 4096, 192)])
def test_grouped_gemm_variants(dtype, rows, N, K):
    from dhellam_amd.operators import moe
    G = len(rows)
    offs = torch.tensor(np.concatenate(([7], 7 + np.cumsum(rows))), dtype=torch.int32)   # non-zero base on purpose
    R = sum(rows)
    a = randn((R, K), dtype, 1, std=0.5)
    b = randn((G, N, K), dtype, 2, std=0.5)
    c = moe.grouped_gemm_nt(a.cuda(), b.cuda(), offs.cuda())
    ref = torch.cat([a[sum(rows[:g]):sum(rows[:g + 1])].double() @ b[g].double().T for g in range(G)])
    assert_close(c, ref, dtype, "NT")
    bt = b.transpose(1, 2).contiguous()   # [G, K, N]
    c2 = moe.grouped_gemm_nn(a.cuda(), bt.cuda(), offs.cuda())
    assert_close(c2, ref, dtype, "NN")
    d = randn((R, N), dtype, 3, std=0.5)
    w = moe.grouped_gemm_tn(d.cuda(), a.cuda(), offs.cuda())
    wref = torch.stack([d[sum(rows[:g]):sum(rows[:g + 1])].double().T @ a[sum(rows[:g]):sum(rows[:g + 1])].double()
                        for g in range(G)])
    assert_close(w, wref, dtype, "TN")
    # rows of a past the last group: the corresponding rows of c come back as zeros (c starts uninitialised)
    a_pad = torch.cat([a, randn((9, K), dtype, 5)]).cuda()
    for fn, bb in ((moe.grouped_gemm_nt, b.cuda()), (moe.grouped_gemm_nn, bt.cuda())):
        torch.empty((R + 9, N), dtype=dtype, device="cuda").fill_(7.0)   # dirty the allocator's next block
        cp = fn(a_pad, bb, offs.cuda())
        assert_close(cp[:R], ref, dtype, "padded")
        assert bool((cp[R:] == 0).all())
    acc0 = randn((G, N, K), dtype, 4)
    acc = acc0.clone().cuda()
    moe.grouped_gemm_tn(d.cuda(), a.cuda(), offs.cuda(), out=acc, accumulate=True)
    assert_close(acc, wref + acc0.double(), dtype, "TN accumulate")


def test_expert_ffn_fwd_bwd():
    from dhellam_amd.operators import moe
    dtype = torch.bfloat16
    T, H, F, E, k = 1024, 512, 768, 8, 2
    lg = _logits(T, E, 9)
    idx, gates, _ = moe.route_topk(lg.cuda(), k)
    plan, _ = moe.sort_assignments(idx, E)
    offs_cpu = plan.expert_offsets.cpu().numpy()
    e_lo, e_hi = 0, 2
    R = int(offs_cpu[e_hi] - offs_cpu[e_lo])
    x = randn((T, H), dtype, 10)
    w1 = randn((2, 2 * F, H), dtype, 11, std=0.02)
    w2 = randn((2, H, F), dtype, 12, std=0.02)
    xp, _ = moe.permute_fwd(x.cuda(), plan, e_lo, e_hi, R)
    offs = plan.expert_offsets[e_lo:e_hi + 1]
    y, saved, _ = moe.expert_ffn_fwd(xp, w1.cuda(), w2.cuda(), offs)
    yo, ho, ao = OM.grouped_ffn(xp.cpu(), w1, w2, offs_cpu[e_lo:e_hi + 1], round_to=dtype)
    assert_close(saved[0], ho, dtype, "h")
    assert_close(y, yo, dtype, "ffn out")
    # backward against autograd of the fp64 oracle, which stores h, a and the gradients that come back through
    # them in the 16-bit type, as the pipeline does
    dy = randn((R, H), dtype, 13)
    xr = xp.cpu().double().requires_grad_()
    w1r, w2r = w1.double().requires_grad_(), w2.double().requires_grad_()
    yr, _, _ = OM.grouped_ffn(xr, w1r, w2r, offs_cpu[e_lo:e_hi + 1], round_to=dtype)
    (yr * dy.double()).sum().backward()
    dxp, dw1, dw2, _ = moe.expert_ffn_bwd(dy.cuda(), xp, w1.cuda(), w2.cuda(), offs, saved)
    assert_close(dxp, xr.grad, dtype, "dxp")
    assert_close(dw1, w1r.grad, dtype, "dw1")
    assert_close(dw2, w2r.grad, dtype, "dw2")
    # ... and the distance to the oracle that rounds nowhere (fp64 throughout): what two 16-bit stores on the way
    # forward and two on the way back may cost, so that a drift of the 16-bit pipeline cannot hide behind an oracle
    # that rounds where the pipeline rounds
    xe = xp.cpu().double().requires_grad_()
    w1e, w2e = w1.double().requires_grad_(), w2.double().requires_grad_()
    ye, _, _ = OM.grouped_ffn(xe, w1e, w2e, offs_cpu[e_lo:e_hi + 1], round_to=None)
    (ye * dy.double()).sum().backward()
    far = {"y": rel_err(y, ye), "dxp": rel_err(dxp, xe.grad), "dw1": rel_err(dw1, w1e.grad), "dw2": rel_err(dw2, w2e.grad)}
    print("expert FFN rel err vs the unrounded oracle:", {k_: f"{v:.2e}" for k_, v in far.items()})
    assert max(far.values()) <= UNROUNDED_BOUND, far


def test_expert_ffn_full_size():
    """The MoE rank share at its full shape (8192 tokens, top-2 of 8 experts, hidden 4096, expert FFN 14336, two
    local experts): forward against the oracle evaluated in fp32 with the 16-bit roundings of h and a, backward
    against fp32 autograd of the same oracle (the gradients that come back through h and a rounded as well).  The oracle's matmuls
    run on the GPU through the library here, a few seconds instead of minutes."""
    from dhellam_amd.operators import moe
    dtype = torch.bfloat16
    T, H, F, E, k = 8192, 4096, 14336, 8, 2
    idx, gates, _ = moe.route_topk(_logits(T, E, 21).cuda(), k)
    plan, _ = moe.sort_assignments(idx, E)
    offs_cpu = plan.expert_offsets.cpu().numpy()
    R = int(offs_cpu[2] - offs_cpu[0])
    assert 3500 < R < 4700
    g = torch.Generator(device="cuda").manual_seed(5)
    rn = lambda *s_, std=1.0: (torch.randn(s_, generator=g, device="cuda") * std).to(dtype)
    x, w1, w2, dy = rn(T, H), rn(2, 2 * F, H, std=0.02), rn(2, H, F, std=0.02), rn(R, H)
    xp, _ = moe.permute_fwd(x, plan, 0, 2, R)
    offs = plan.expert_offsets[0:3]
    y, saved, _ = moe.expert_ffn_fwd(xp, w1, w2, offs)
    yo, ho, _ = OM.grouped_ffn(xp, w1, w2, offs_cpu[0:3], dtype=torch.float32, round_to=dtype)
    assert_close(saved[0], ho, dtype, "h")
    assert_close(y, yo, dtype, "ffn out")
    del yo, ho
    xr = xp.float().requires_grad_()
    w1r, w2r = w1.float().requires_grad_(), w2.float().requires_grad_()
    yr, _, _ = OM.grouped_ffn(xr, w1r, w2r, offs_cpu[0:3], dtype=torch.float32, round_to=dtype)
    (yr * dy.float()).sum().backward()
    dxp, dw1, dw2, _ = moe.expert_ffn_bwd(dy, xp, w1, w2, offs, saved)
    assert_close(dxp, xr.grad, dtype, "dxp")
    assert_close(dw1, w1r.grad, dtype, "dw1")
    assert_close(dw2, w2r.grad, dtype, "dw2")
    # ... and the distance to the same oracle without any rounding of h and a (fp32 throughout)
    del xr, w1r, w2r, yr
    xe = xp.float().requires_grad_()
    w1e, w2e = w1.float().requires_grad_(), w2.float().requires_grad_()
    ye, _, _ = OM.grouped_ffn(xe, w1e, w2e, offs_cpu[0:3], dtype=torch.float32, round_to=None)
    (ye * dy.float()).sum().backward()
    far = {"y": rel_err(y, ye), "dxp": rel_err(dxp, xe.grad), "dw1": rel_err(dw1, w1e.grad), "dw2": rel_err(dw2, w2e.grad)}
    print("expert FFN (full size) rel err vs the unrounded oracle:", {k_: f"{v:.2e}" for k_, v in far.items()})
    assert max(far.values()) <= UNROUNDED_BOUND, far


def test_expert_ffn_is_deterministic():
    """Two runs on the same inputs give the same bits (no atomics, fixed reduction orders), forward and backward."""
    from dhellam_amd.operators import moe
    dtype = torch.bfloat16
    T, H, F, E, k = 4096, 1024, 1536, 8, 2
    idx, gates, _ = moe.route_topk(_logits(T, E, 31).cuda(), k)
    plan, _ = moe.sort_assignments(idx, E)
    R = int((plan.expert_offsets[3] - plan.expert_offsets[0]).item())
    x, dy = randn((T, H), dtype, 1).cuda(), randn((R, H), dtype, 2).cuda()
    w1, w2 = randn((3, 2 * F, H), dtype, 3, std=0.02).cuda(), randn((3, H, F), dtype, 4, std=0.02).cuda()
    offs = plan.expert_offsets[0:4]
    runs = []
    for _ in range(2):
        xp, _ = moe.permute_fwd(x, plan, 0, 3, R)
        y, saved, _ = moe.expert_ffn_fwd(xp, w1, w2, offs)
        dxp, dw1, dw2, _ = moe.expert_ffn_bwd(dy, xp, w1, w2, offs, saved)
        out, _ = moe.unpermute_fwd(y, plan, gates, 0, 3)
        runs.append((y, dxp, dw1, dw2, out))
    for a, b in zip(*runs):
        assert torch.equal(a, b)


def test_offsets_past_the_callers_bound_touch_nothing_beyond_it():
    """The row counts live on the device, so the caller cannot check them against its buffers: whatever
    ``expert_offsets`` says, the gather and the grouped GEMMs write no row past ``max_rows`` (guard rows behind
    the buffers stay intact) and every kernel ends normally."""
    from dhellam_amd import _lib
    lib = _lib.load()
    T, H, E, k, N = 512, 256, 4, 2, 256
    dt = torch.bfloat16
    idx = torch.from_numpy(np.random.default_rng(0).integers(0, E, size=(T, k), dtype=np.int32)).cuda()
    from dhellam_amd.operators import moe
    plan, _ = moe.sort_assignments(idx, E)
    R = T * k                       # rows of all experts together
    max_rows, guard = 300, 64       # the caller's (too small) bound
    st = torch.cuda.current_stream().cuda_stream
    x = randn((T, H), dt, 1).cuda()
    buf = torch.full((max_rows + guard, H), 3.0, dtype=dt, device="cuda")
    _lib.check(lib.dh_moe_gather_rows(x.data_ptr(), plan.sorted_idx.data_ptr(), None, buf.data_ptr(),
                                      plan.expert_offsets.data_ptr(), 0, E, max_rows, k, H, _lib.dt(x), st))
    torch.cuda.synchronize()
    assert (buf[max_rows:] == 3.0).all(), "gather wrote past max_rows"
    want = x[(plan.sorted_idx[:max_rows] // k).long()]
    assert torch.equal(buf[:max_rows], want)
    # grouped GEMMs: a holds max_rows rows, offsets describe R > max_rows rows
    a = randn((max_rows, H), dt, 2, std=0.5).cuda()
    b = randn((E, N, H), dt, 3, std=0.5).cuda()
    offs_np = plan.expert_offsets.cpu().numpy()
    for name, fn, bb in (("nt", lib.dh_grouped_gemm_nt, b), ("nn", lib.dh_grouped_gemm_nn, b.transpose(1, 2).contiguous())):
        c = torch.full((max_rows + guard, N), 3.0, dtype=dt, device="cuda")
        _lib.check(fn(a.data_ptr(), bb.data_ptr(), c.data_ptr(), plan.expert_offsets.data_ptr(), E, max_rows, N, H,
                      _lib.dt(a), None, 0, st))
        torch.cuda.synchronize()
        assert (c[max_rows:] == 3.0).all(), f"grouped GEMM {name} wrote past max_rows"
        ref = torch.zeros((max_rows, N), dtype=torch.float64)
        for g in range(E):
            lo, hi = min(int(offs_np[g]), max_rows), min(int(offs_np[g + 1]), max_rows)
            ref[lo:hi] = a[lo:hi].cpu().double() @ b[g].cpu().double().T
        assert_close(c[:max_rows], ref, dt, f"grouped GEMM {name}, rows cut off at max_rows")
    # wgrad: the reduction runs over the rows that exist only
    dw = torch.empty((E, H, N), dtype=dt, device="cuda")
    cc = randn((max_rows, N), dt, 4, std=0.5).cuda()
    _lib.check(lib.dh_grouped_gemm_tn(a.data_ptr(), cc.data_ptr(), dw.data_ptr(), plan.expert_offsets.data_ptr(), E,
                                      max_rows, H, N, 0, _lib.dt(a), st))
    torch.cuda.synchronize()
    ref = torch.zeros((E, H, N), dtype=torch.float64)
    for g in range(E):
        lo, hi = min(int(offs_np[g]), max_rows), min(int(offs_np[g + 1]), max_rows)
        ref[g] = a[lo:hi].cpu().double().T @ cc[lo:hi].cpu().double()
    assert_close(dw, ref, dt, "grouped GEMM tn, rows cut off at max_rows")
    assert R > max_rows


def test_sort_leaves_out_expert_ids_outside_the_range():
    """An id < 0 or >= E (a foreign router's bug) is not counted and gets dest_row -1; the others are sorted as if
    it were not there."""
    from dhellam_amd.operators.moe import sort_assignments
    rng = np.random.default_rng(1)
    E = 8
    idx = rng.integers(0, E, size=(3000, 2), dtype=np.int32)
    bad = rng.random(idx.shape) < 0.01
    idx_bad = idx.copy()
    idx_bad[bad] = np.where(rng.random(bad.sum()) < 0.5, -3, E + 5)
    plan, _ = sort_assignments(torch.from_numpy(idx_bad).cuda(), E)
    flat, keep = idx_bad.reshape(-1), ~bad.reshape(-1)
    tpe = np.bincount(flat[keep], minlength=E)
    assert np.array_equal(plan.tokens_per_expert.cpu().numpy(), tpe)
    order = np.flatnonzero(keep)[np.argsort(flat[keep], kind="stable")]
    n_good = int(keep.sum())
    assert np.array_equal(plan.sorted_idx.cpu().numpy()[:n_good], order)
    dest = plan.dest_row.cpu().numpy()
    assert (dest[~keep] == -1).all()
    assert np.array_equal(dest[order], np.arange(n_good))

def test_expert_ffn_bwd_with_resident_weight_transposes():
    """Expert weights registered with keep_transposed: the data gradients run as NT products against [G, K, N]
    copies and give the bits of the NN products; the copies follow an in-place update of the weights."""
    from dhellam_amd import _Clib
    from dhellam_amd.operators import moe
    dt = torch.bfloat16
    G, H, F, R = 3, 256, 512, 700
    offs = torch.tensor([0, 300, 300, 700], dtype=torch.int32).cuda()           # one empty expert
    xp, dy = randn((R, H), dt, 1).cuda(), randn((R, H), dt, 2).cuda()
    w1, w2 = randn((G, 2 * F, H), dt, 3, std=0.05).cuda(), randn((G, H, F), dt, 4, std=0.05).cuda()
    y, saved, _ = moe.expert_ffn_fwd(xp, w1, w2, offs)
    ref = moe.expert_ffn_bwd(dy, xp, w1, w2, offs, saved)
    w1t, w2t = _Clib.keep_transposed(w1), _Clib.keep_transposed(w2)
    assert w1t.shape == (G, H, 2 * F) and torch.equal(w2t, w2.transpose(1, 2).contiguous())
    got = moe.expert_ffn_bwd(dy, xp, w1, w2, offs, saved)
    for a, b in zip(ref[:3], got[:3]):
        assert torch.equal(a, b)
    w2.mul_(0.5)
    assert torch.equal(_Clib.transposed_of(w2), w2.transpose(1, 2).contiguous())


@pytest.mark.parametrize("form,K,N,last", [("nt", 192, 4096, 500), ("nt", 1024, 4096, 500), ("nn", 192, 4096, 500),
                                           ("nn", 1024, 4096, 500),
                                           ("nt", 320, 4232, 500),    # n ends inside a tile: 4232 = 16 * 256 + 136
                                           ("nt", 256, 4096, 10), ("nn", 256, 4096, 10),    # groups end before max_rows
                                           ("nt", 192, 8192, 500), ("nn", 320, 8192, 500)]) # two full rounds, then a split one
def test_grouped_gemm_split_last_round(form, K, N, last):
    """The chip-filling kernels through the C ABI, with and without a workspace (last round split along k / one workgroup per tile):
    both within the bound of the fp64 product, the split result the same on every run, rows cut off at max_rows
    (the offsets describe more rows than the operands hold), nothing written past them; rows between the last
    group's end and max_rows come back as zeros (the output starts out as 3.0 everywhere)."""
    from dhellam_amd import _lib
    lib = _lib.load()
    dt = torch.bfloat16
    rows = [2100, 0, 1990, 37, last]
    G, R = len(rows), sum(rows)
    max_rows, guard = 4200, 64                      # last = 500: the last group is cut off, 73 of its rows exist
    offs_np = np.concatenate(([5], 5 + np.cumsum(rows))).astype(np.int32)
    offs = torch.from_numpy(offs_np).cuda()
    a = randn((max_rows, K), dt, 11, std=0.5).cuda()
    b = randn((G, N, K), dt, 12, std=0.5).cuda()
    bb = b if form == "nt" else b.transpose(1, 2).contiguous()
    fn = lib.dh_grouped_gemm_nt if form == "nt" else lib.dh_grouped_gemm_nn
    st = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(lib.dh_grouped_gemm_workspace_bytes(), dtype=torch.uint8, device="cuda")
    ref = torch.zeros((max_rows, N), dtype=torch.float64)
    for g in range(G):
        lo, hi = min(int(offs_np[g]) - 5, max_rows), min(int(offs_np[g + 1]) - 5, max_rows)
        ref[lo:hi] = a[lo:hi].cpu().double() @ b[g].cpu().double().T
    outs = []
    for wsp, nbytes in ((None, 0), (ws.data_ptr(), ws.numel()), (ws.data_ptr(), ws.numel())):
        ws.fill_(0x7f)                              # the workspace's contents on entry do not matter
        c = torch.full((max_rows + guard, N), 3.0, dtype=dt, device="cuda")
        _lib.check(fn(a.data_ptr(), bb.data_ptr(), c.data_ptr(), offs.data_ptr(), G, max_rows, N, K, _lib.dt(a),
                      wsp, nbytes, st))
        torch.cuda.synchronize()
        assert (c[max_rows:] == 3.0).all(), "wrote past max_rows"
        assert_close(c[:max_rows], ref, dt, f"grouped GEMM {form}, workspace {nbytes}")
        outs.append(c)
    assert torch.equal(outs[1], outs[2]), "split result differs between runs"
    # a workspace that is too small is not used (the product falls back to one workgroup per tile)
    c = torch.full((max_rows + guard, N), 3.0, dtype=dt, device="cuda")
    _lib.check(fn(a.data_ptr(), bb.data_ptr(), c.data_ptr(), offs.data_ptr(), G, max_rows, N, K, _lib.dt(a),
                  ws.data_ptr(), 1 << 20, st))
    torch.cuda.synchronize()
    assert torch.equal(c, outs[0])


@pytest.mark.parametrize("form", ["nt", "nn"])
def test_grouped_gemm_sixty_four_groups(form):
    """The largest group count the kernels take (one group per lane of the workgroup's group table), on the
    chip-filling kernels: groups of 0 to 130 rows, most of them one partial tile, a first offset that is not 0."""
    from dhellam_amd.operators import moe
    dt = torch.bfloat16
    rng = np.random.default_rng(5)
    rows = rng.integers(0, 131, size=64)
    rows[7] = 0
    rows[63] = 130
    R, K, N = int(rows.sum()), 192, 4096
    offs_np = np.concatenate(([11], 11 + np.cumsum(rows))).astype(np.int32)
    offs = torch.from_numpy(offs_np).cuda()
    a = randn((R, K), dt, 31, std=0.5).cuda()
    b = randn((64, N, K), dt, 32, std=0.5).cuda()
    ref = torch.zeros((R, N), dtype=torch.float64)
    st = np.concatenate(([0], np.cumsum(rows)))
    for g in range(64):
        ref[st[g]:st[g + 1]] = a[st[g]:st[g + 1]].cpu().double() @ b[g].cpu().double().T
    if form == "nt":
        c = moe.grouped_gemm_nt(a, b, offs)
    else:
        c = moe.grouped_gemm_nn(a, b.transpose(1, 2).contiguous(), offs)
    assert_close(c, ref, dt, f"64 groups, {form}")


@pytest.mark.parametrize("dtype,M,N", [(torch.bfloat16, 4096, 2048), (torch.float16, 4096, 2048),
                                       (torch.bfloat16, 2304, 7424)])    # 9 x 29 tiles: a last band of one m tile, odd counts
def test_grouped_gemm_tn_chip_filling(dtype, M, N):
    """Weight-gradient products large enough for the 256x256-tile kernel (m, n multiples of 256, >= 256 tiles): an
    empty group (its output must be zeros), groups of 1, 65 and 300 rows (k not a multiple of the 64-deep slice),
    rows of the operands past the last group (not read), accumulation into an existing output, same result twice."""
    from dhellam_amd.operators import moe
    rows = [300, 0, 65, 1]
    G, R = len(rows), sum(rows)
    offs = torch.tensor(np.concatenate(([3], 3 + np.cumsum(rows))), dtype=torch.int32).cuda()
    a = randn((R + 7, M), dtype, 21, std=0.5).cuda()
    b = randn((R + 7, N), dtype, 22, std=0.5).cuda()
    st = np.concatenate(([0], np.cumsum(rows)))
    ref = torch.stack([a[st[g]:st[g + 1]].cpu().double().T @ b[st[g]:st[g + 1]].cpu().double() for g in range(G)])
    w = moe.grouped_gemm_tn(a, b, offs)
    assert_close(w, ref, dtype, "TN")
    assert bool((w[1] == 0).all()), "empty group"
    assert torch.equal(w, moe.grouped_gemm_tn(a, b, offs))
    acc0 = randn((G, M, N), dtype, 23)
    acc = acc0.clone().cuda()
    moe.grouped_gemm_tn(a, b, offs, out=acc, accumulate=True)
    assert_close(acc, ref + acc0.double(), dtype, "TN accumulate")
    assert torch.equal(acc[1].cpu(), acc0[1]), "accumulating an empty group must leave the output as it was"
