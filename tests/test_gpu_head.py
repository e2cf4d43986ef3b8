"""GPU parity of the head-block operators (word embedding, vocab-parallel cross entropy, masked mean,
and the head block built from them) against the CPU oracle in fp64, on the same seeded inputs already
rounded to the run dtype.  Tolerances: rel-err <= 1e-5 (fp32), <= 1e-2 (bf16 / fp16); index outputs
(target mask, local target index) bit-exact.
"""
import pytest
import torch

from oracle import head as OH
from oracle import ops as O
from tests.util import assert_close, randn

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


@pytest.fixture
def tp():
    from dhellam_amd.common import parallel_state as ps
    yield ps.set_tensor_model_parallel
    ps.set_tensor_model_parallel(0, 1)


def _targets(shape, lo, hi, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi, shape, generator=g, dtype=torch.int64)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,rank,world", [((64, 16032), 0, 1), ((4, 9, 1000), 0, 1), ((33, 16032), 3, 8),
                                              ((5, 70000), 1, 2), ((3, 131080), 0, 1), ((2, 140003), 0, 1), ((7, 37), 0, 1), ((3, 1), 0, 1),
                                              ((0, 64), 0, 1)])
@pytest.mark.parametrize("ls", [0.0, 0.1])
@pytest.mark.parametrize("keep", [True, False])
def test_cross_entropy(tp, dtype, shape, rank, world, ls, keep):
    from dhellam_amd.operators.loss import cross_entropy_bwd, cross_entropy_fwd
    cols = shape[-1]
    if ls > 0 and cols == 1:
        pytest.skip("label smoothing needs two classes")
    tp(rank, world)
    x = randn(shape, dtype, 1, std=3.0)
    t = _targets(shape[:-1], 0, cols * world, 2)
    if t.numel() > 2:
        t.view(-1)[0], t.view(-1)[1] = rank * cols, rank * cols + cols - 1     # both ends of this rank's slice
    dout = randn(shape[:-1], torch.float32, 3)
    ref = OH.cross_entropy_fwd([x], t, ls, collectives=False, ranks=[rank])[0]
    inputs = {"vocab_parallel_logits": x.cuda(), "target": t.cuda()}
    out = cross_entropy_fwd(inputs, ls, keep_softmax=keep)
    assert out["vocab_size"] == cols and out["label_smoothing"] == ls
    assert torch.equal(out["target_mask"].cpu(), ref["target_mask"])
    assert torch.equal(out["masked_target_1d"].cpu(), ref["masked_target_1d"])
    if t.numel() == 0:
        return
    assert_close(out["loss"], ref["loss"], torch.float32, "loss")
    assert_close(out["row_max"], ref["row_max"].reshape(-1), torch.float32, "row_max")
    assert_close(out["sum_exp"], ref["sum_exp"].reshape(-1), torch.float32, "sum_exp")
    assert_close(out["predicted"], ref["predicted"], torch.float32, "predicted")
    if keep:
        assert_close(out["softmax"], ref["softmax"], dtype, "softmax")
    else:
        assert out["softmax"] is None
    # the oracle's backward from the oracle's own softmax; ours from what our forward kept
    gref = OH.cross_entropy_bwd(ref, dout)
    g = cross_entropy_bwd([inputs, out], dout.cuda())
    assert g.shape == x.shape and g.dtype == dtype
    assert_close(g, gref, dtype, "grad")
    if keep:
        assert g.data_ptr() == out["softmax"].data_ptr()       # in place, as in the reference


def test_cross_entropy_strided_rows_and_in_place_over_logits(tp):
    """Rows with a pitch (a column block of a wider matrix, 16-byte alignment broken) and the gradient
    written over the logits."""
    from dhellam_amd.operators.loss import cross_entropy_bwd, cross_entropy_fwd
    wide = randn((50, 1003), torch.bfloat16, 5, std=2.0)
    x = wide[:, 1:1001]
    t = _targets((50,), 0, 1000, 6)
    ref = OH.cross_entropy_fwd([x], t)[0]
    xc = wide.cuda()[:, 1:1001]
    inputs = {"vocab_parallel_logits": xc, "target": t.cuda()}
    out = cross_entropy_fwd(inputs, 0.0, keep_softmax=False)
    assert_close(out["loss"], ref["loss"], torch.float32, "loss")
    dout = randn((50,), torch.float32, 7)
    g = cross_entropy_bwd([inputs, out], dout.cuda(), grad_out=xc)
    assert g.data_ptr() == xc.data_ptr()
    assert_close(xc, OH.cross_entropy_bwd(ref, dout), torch.bfloat16, "grad over logits")


def test_cross_entropy_in_place_equals_out_of_place():
    """Short rows, many of them: the gradient written over the logits must be bit-identical to the one written
    to a new tensor (the target's element is read before any wavefront of the row stores)."""
    from dhellam_amd.operators.loss import cross_entropy_bwd, cross_entropy_fwd
    for dtype, cols in ((torch.float32, 512), (torch.bfloat16, 1536), (torch.bfloat16, 40)):
        x = randn((8192, cols), dtype, 11, std=2.0).cuda()
        t = _targets((8192,), 0, cols, 12).cuda()
        dout = randn((8192,), torch.float32, 13).cuda()
        inputs = {"vocab_parallel_logits": x, "target": t}
        out = cross_entropy_fwd(inputs, 0.0, keep_softmax=False)
        g1 = cross_entropy_bwd([inputs, out], dout)
        for _ in range(3):
            xc = x.clone()
            inputs2 = {"vocab_parallel_logits": xc, "target": t}
            g2 = cross_entropy_bwd([inputs2, out], dout, grad_out=xc)
            assert torch.equal(g1, g2)


def test_cross_entropy_extreme_logits():
    """Large offsets and a dominant class: the max shift keeps everything finite."""
    from dhellam_amd.operators.loss import cross_entropy_fwd
    x = randn((8, 512), torch.float32, 9)
    x[0] += 1e4
    x[1] -= 1e4
    x[2, 7] = 200.0
    x[3, :] = -50.0
    t = torch.tensor([0, 1, 7, 5, 3, 2, 1, 0])
    ref = OH.cross_entropy_fwd([x], t)[0]
    out = cross_entropy_fwd({"vocab_parallel_logits": x.cuda(), "target": t.cuda()}, 0.0)
    assert torch.isfinite(out["loss"]).all() and torch.isfinite(out["softmax"]).all()
    assert_close(out["loss"], ref["loss"], torch.float32, "loss")
    assert_close(out["softmax"], ref["softmax"], torch.float32, "softmax")


def test_cross_entropy_rejects_bad_arguments():
    from dhellam_amd.operators.loss import cross_entropy_fwd
    x, t = torch.zeros(4, 8, device="cuda"), torch.zeros(4, dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError):
        cross_entropy_fwd({"vocab_parallel_logits": x, "target": t}, 1.5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_shape,hidden,rows,rank,world", [((2, 64), 8192, 500, 0, 1), ((1, 4096), 1024, 16032, 2, 8),
                                                            ((3, 5), 24, 7, 1, 4), ((1, 300), 16384, 3, 0, 1), ((0,), 64, 4, 0, 1)])
def test_word_embedding(tp, dtype, n_shape, hidden, rows, rank, world):
    from dhellam_amd.operators.embedding import word_embedding_bwd, word_embedding_fwd
    tp(rank, world)
    table = randn((rows, hidden), dtype, 1)
    ids = _targets(n_shape, 0, rows * world, 2)
    if ids.numel() > 4:
        ids.view(-1)[:4] = torch.tensor([rank * rows, rank * rows + rows - 1, rank * rows, rank * rows])
    dout = randn((*n_shape, hidden), dtype, 3)
    tc = table.cuda()
    inputs = {"vocab": tc, "token_ids": ids.cuda()}
    out = word_embedding_fwd(inputs)
    ref = OH.word_embedding_fwd(table, ids, rank, world)
    assert torch.equal(out["word_embeddings"].cpu().double(), ref)                 # a gather: exact
    # backward: accumulates into .grad (16-bit, one rounding of old + fp32 sum) and into an fp32 main_grad
    g0 = randn((rows, hidden), dtype, 4)
    tc.grad = g0.clone().cuda()
    assert word_embedding_bwd([inputs, out], dout.cuda()) is None
    gref = OH.word_embedding_bwd(dout, ids, rows, rank, world)
    assert_close(tc.grad, g0.double() + gref, dtype, "grad")
    tc.main_grad = torch.zeros(rows, hidden, dtype=torch.float32, device="cuda")
    word_embedding_bwd([inputs, out], dout.cuda())
    assert_close(tc.main_grad, gref, torch.float32, "main_grad")
    again = tc.main_grad.clone()
    tc.main_grad.zero_()
    word_embedding_bwd([inputs, out], dout.cuda())
    assert torch.equal(tc.main_grad, again)                                        # deterministic


def test_word_embedding_all_positions_one_id():
    """Every position holds the same id: one block sums thousands of rows in order."""
    from dhellam_amd.operators.embedding import word_embedding_bwd, word_embedding_fwd
    table = randn((4, 256), torch.bfloat16, 1).cuda()
    ids = torch.full((1, 1500), 2, dtype=torch.int64)
    dout = randn((1, 1500, 256), torch.bfloat16, 2)
    inputs = {"vocab": table, "token_ids": ids.cuda()}
    table.main_grad = torch.zeros(4, 256, dtype=torch.float32, device="cuda")
    word_embedding_bwd([inputs, word_embedding_fwd(inputs)], dout.cuda())
    assert_close(table.main_grad, OH.word_embedding_bwd(dout, ids, 4), torch.float32, "main_grad")


@pytest.mark.parametrize("n", [1, 37, 4096, 70001])
def test_mask_scale_loss(n):
    from dhellam_amd.operators.loss import mask_scale_loss_bwd, mask_scale_loss_fwd
    losses = randn((1, n), torch.float32, 1).abs()
    mask = (_targets((1, n), 0, 2, 2) if n > 1 else torch.ones(1, 1, dtype=torch.int64))
    mask[0, 0] = 1
    inputs = {"loss_mask": mask.cuda(), "output_tensor": losses.cuda(), "num_microbatch": 4, "loss_scale": 1024.0}
    out = mask_scale_loss_fwd(inputs)
    assert out["loss"].dim() == 0
    assert_close(out["loss"], OH.mask_scale_loss_fwd(losses, mask, 4, 1024.0), torch.float32, "loss")
    g = mask_scale_loss_bwd([inputs, out], None)
    assert g.shape == losses.shape
    assert_close(g, OH.mask_scale_loss_bwd(losses, mask, 4, 1024.0), torch.float32, "grad")


@pytest.mark.parametrize("dtype,tol_scale", [(torch.float32, 30), (torch.bfloat16, 2)])
@pytest.mark.parametrize("ln", [False, True])
def test_head_block(tp, dtype, tol_scale, ln):
    """pre_process -> post_process -> backward of both against fp64 autograd through the oracle's operators."""
    from dhellam_amd.core import dshb
    tp(0, 1)
    s, b, h, v = 96, 2, 256, 1000
    table = randn((v, h), dtype, 1, std=0.05)
    gamma = (1 + 0.1 * randn((h,), torch.float32, 2)).to(dtype)
    beta = randn((h,), dtype, 3, std=0.1) if ln else None
    ids, labels = _targets((b, s), 0, v, 4), _targets((b, s), 0, v, 5)
    mask = _targets((b, s), 0, 2, 6)
    # oracle: fp64 autograd over embedding -> (layers: identity) -> norm -> logits -> CE -> masked mean
    tr, gr = table.double().requires_grad_(True), gamma.double().requires_grad_(True)
    br = beta.double().requires_grad_(True) if ln else None
    hid = OH.word_embedding_fwd(tr, ids).transpose(0, 1)
    y, _, _ = O.norm_fwd(hid, gr, br, 1e-5)
    # the HIP path rounds ln_out and the logits to the run dtype; the oracle mirrors those two roundings
    rt = (lambda z: z + (z.detach().to(dtype).double() - z.detach()))
    logits = rt(rt(y) @ tr.t())
    tl = OH.cross_entropy_fwd([logits], labels.transpose(0, 1))[0]["loss"].transpose(0, 1)
    loss_ref = OH.mask_scale_loss_fwd(tl, mask, 4, 2.0)
    loss_ref.backward()

    tc, gc = table.cuda(), gamma.cuda()
    bc = beta.cuda() if ln else None
    for p in (tc, gc, bc):
        if p is not None:
            p.main_grad = torch.zeros_like(p, dtype=torch.float32)
    hidden, ectx = dshb.pre_process(ids.cuda(), tc)
    assert hidden.shape == (s, b, h)
    loss, ctx = dshb.post_process(hidden, gc, bc, labels.cuda(), mask.cuda(), tc, 4, 2.0)
    assert_close(loss, loss_ref.detach(), torch.float32, "loss")
    d_hidden = dshb.post_process_bwd(ctx)
    dshb.pre_process_bwd(ectx, d_hidden)
    assert_close(tc.main_grad, tr.grad, dtype, "table grad")
    assert_close(gc.main_grad, gr.grad, dtype, "gamma grad")
    if ln:
        assert_close(bc.main_grad, br.grad, dtype, "beta grad")
