"""MoE routing, token permute/unpermute and the grouped expert FFN for one
expert-parallel rank.

The reference has no MoE; these operators follow its wrapper convention
(``stream=None`` means the current stream, trailing elapsed-ms return) and the
dropless top-k semantics of Mixtral / Megatron-core.  All row counts stay on the
device (``MoEPlan.expert_offsets``): nothing here synchronises with the host, so
buffers are sized by the caller-provided ``max_rows`` bound.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import _lib
from .._Clib import _note_read, transposed_of
from ._util import on_stream


@dataclass
class MoEPlan:
    """Result of sorting the flat (token, slot) assignment list by expert."""
    tokens: int
    k: int
    num_experts: int
    tokens_per_expert: torch.Tensor   # int32 [E]
    expert_offsets: torch.Tensor      # int32 [E + 1]
    sorted_idx: torch.Tensor          # int32 [T * k], assignment ids in sorted order
    dest_row: torch.Tensor            # int32 [T * k], sorted position of each assignment


def route_topk(logits, k, stream=None, profiling=False):
    """logits fp32 [T, E] -> (topk_idx int32 [T, k], gates fp32 [T, k], ms).  Descending
    logit, ties to the lower expert id; gates = softmax over the k selected logits."""
    assert logits.is_cuda and logits.dtype == torch.float32 and logits.is_contiguous() and logits.dim() == 2
    lib = _lib.load()
    t, e = logits.shape
    el: list = []
    with on_stream(stream, profiling, el) as st:
        idx = torch.empty((t, k), dtype=torch.int32, device=logits.device)
        gates = torch.empty((t, k), dtype=torch.float32, device=logits.device)
        _lib.check(lib.dh_moe_route_topk(logits.data_ptr(), idx.data_ptr(), gates.data_ptr(), t, e, k, st.cuda_stream))
    return idx, gates, el[0]


def sort_assignments(topk_idx, num_experts, stream=None, profiling=False):
    """Stable counting sort of the assignments by expert id -> (MoEPlan, ms)."""
    assert topk_idx.is_cuda and topk_idx.dtype == torch.int32 and topk_idx.is_contiguous()
    lib = _lib.load()
    t, k = topk_idx.shape
    n = t * k
    dev = topk_idx.device
    el: list = []
    with on_stream(stream, profiling, el) as st:
        tpe = torch.empty(num_experts, dtype=torch.int32, device=dev)
        offs = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
        sorted_idx = torch.empty(n, dtype=torch.int32, device=dev)
        dest = torch.empty(n, dtype=torch.int32, device=dev)
        ws = torch.empty(lib.dh_moe_sort_workspace_bytes(n, num_experts), dtype=torch.uint8, device=dev)
        _lib.check(lib.dh_moe_sort(topk_idx.data_ptr(), tpe.data_ptr(), offs.data_ptr(), sorted_idx.data_ptr(),
                                   dest.data_ptr(), ws.data_ptr(), ws.numel(), n, num_experts, st.cuda_stream))
    return MoEPlan(t, k, num_experts, tpe, offs, sorted_idx, dest), el[0]


def _gather(x, plan, e_lo, e_hi, max_rows, row_scale, stream, profiling):
    lib = _lib.load()
    assert x.is_cuda and x.is_contiguous() and x.dim() == 2
    el: list = []
    with on_stream(stream, profiling, el) as st:
        out = torch.empty((max_rows, x.shape[1]), dtype=x.dtype, device=x.device)   # the kernel zeroes the unused rows
        _lib.check(lib.dh_moe_gather_rows(x.data_ptr(), plan.sorted_idx.data_ptr(), _lib.ptr(row_scale),
                                          out.data_ptr(), plan.expert_offsets.data_ptr(), e_lo, e_hi, max_rows,
                                          plan.k, x.shape[1], _lib.dt(x), st.cuda_stream))
    return out, el[0]


def _scatter(y, plan, e_lo, e_hi, gates, stream, profiling):
    lib = _lib.load()
    assert y.is_cuda and y.is_contiguous() and y.dim() == 2
    el: list = []
    with on_stream(stream, profiling, el) as st:
        out = torch.empty((plan.tokens, y.shape[1]), dtype=y.dtype, device=y.device)
        _lib.check(lib.dh_moe_scatter_rows(y.data_ptr(), plan.dest_row.data_ptr(), _lib.ptr(gates), out.data_ptr(),
                                           plan.expert_offsets.data_ptr(), e_lo, e_hi, plan.tokens, plan.k,
                                           y.shape[1], _lib.dt(y), st.cuda_stream))
    return out, el[0]


def permute_fwd(x, plan, e_lo, e_hi, max_rows, stream=None, profiling=False):
    """x [T, H] -> (permuted [max_rows, H], ms): the rows routed to local experts
    [e_lo, e_hi), grouped by expert, original (token, slot) order inside an expert.
    Rows past the real count are zero."""
    return _gather(x, plan, e_lo, e_hi, max_rows, None, stream, profiling)


def permute_bwd(d_permuted, plan, e_lo, e_hi, stream=None, profiling=False):
    """Gradient of permute_fwd: dx[t] = sum of the local rows that came from token t."""
    return _scatter(d_permuted, plan, e_lo, e_hi, None, stream, profiling)


def unpermute_fwd(y, plan, gates, e_lo, e_hi, stream=None, profiling=False):
    """y [rows, H] (expert outputs, permuted order), gates fp32 [T, k] ->
    (out [T, H], ms) with out[t] = sum_j gates[t, j] * y[row(t, j)] over local assignments."""
    assert gates.dtype == torch.float32 and gates.is_contiguous()
    return _scatter(y, plan, e_lo, e_hi, gates, stream, profiling)


def unpermute_bwd(dout, y, plan, gates, e_lo, e_hi, max_rows, stream=None, profiling=False):
    """Returns (dy [max_rows, H], dgates fp32 [T, k], ms): dy[r] = gate * dout[token(r)],
    dgates[t, j] = <dout[t], y[row(t, j)]> (0 for assignments owned by other ranks)."""
    lib = _lib.load()
    el: list = []
    with on_stream(stream, profiling, el) as st:
        dy, _ = _gather(dout, plan, e_lo, e_hi, max_rows, gates, st, False)
        dgates = torch.empty((plan.tokens, plan.k), dtype=torch.float32, device=dout.device)
        _lib.check(lib.dh_moe_gate_grad(dout.data_ptr(), y.data_ptr(), plan.dest_row.data_ptr(), dgates.data_ptr(),
                                        plan.expert_offsets.data_ptr(), e_lo, e_hi, plan.tokens, plan.k,
                                        dout.shape[1], _lib.dt(dout), st.cuda_stream))
    return dy, dgates, el[0]


# ---------------------------------------------------------------------------------------
# grouped GEMM and the expert FFN built from it
# ---------------------------------------------------------------------------------------
_gg_workspaces: dict = {}


def _gg_workspace(rows, n, device, stream):
    """(pointer, bytes) of the split-k workspace for a product of this size on this stream: one buffer per
    (device, stream), since calls on different streams may overlap.  Small products (fewer 256x256 tiles than
    compute units) do not use one."""
    if -(-rows // 256) * -(-n // 256) < 256:
        return None, 0
    key = (device, stream.cuda_stream)
    ws = _gg_workspaces.get(key)
    if ws is None:
        ws = torch.empty(_lib.load().dh_grouped_gemm_workspace_bytes(), dtype=torch.uint8, device=device)
        _gg_workspaces[key] = ws
    return ws.data_ptr(), ws.numel()


def grouped_gemm_nt(a, b, offs, max_rows=None, out=None, stream=None):
    """c[rows_g] = a[rows_g] @ b[g].T ; a [R, K], b [G, N, K] -> c [R, N]."""
    lib = _lib.load()
    g, n, k = b.shape
    assert a.is_contiguous() and b.is_contiguous() and a.shape[1] == k and offs.numel() == g + 1
    st = stream or torch.cuda.current_stream()
    with torch.cuda.stream(st):
        # rows past the last group are zeroed by the library; everything else is written
        c = out if out is not None else torch.empty((a.shape[0], n), dtype=a.dtype, device=a.device)
        if out is None and max_rows is not None and max_rows < a.shape[0]:
            c[max_rows:].zero_()
        rows = a.shape[0] if max_rows is None else max_rows
        ws, ws_bytes = _gg_workspace(rows, n, a.device, st)
        _lib.check(lib.dh_grouped_gemm_nt(a.data_ptr(), b.data_ptr(), c.data_ptr(), offs.data_ptr(), g, rows, n, k,
                                          _lib.dt(a), ws, ws_bytes, st.cuda_stream))
    return c


def grouped_gemm_nn(a, b, offs, max_rows=None, out=None, stream=None):
    """c[rows_g] = a[rows_g] @ b[g] ; a [R, K], b [G, K, N] -> c [R, N]."""
    lib = _lib.load()
    g, k, n = b.shape
    assert a.is_contiguous() and b.is_contiguous() and a.shape[1] == k and offs.numel() == g + 1
    st = stream or torch.cuda.current_stream()
    with torch.cuda.stream(st):
        # rows past the last group are zeroed by the library; everything else is written
        c = out if out is not None else torch.empty((a.shape[0], n), dtype=a.dtype, device=a.device)
        if out is None and max_rows is not None and max_rows < a.shape[0]:
            c[max_rows:].zero_()
        rows = a.shape[0] if max_rows is None else max_rows
        ws, ws_bytes = _gg_workspace(rows, n, a.device, st)
        _lib.check(lib.dh_grouped_gemm_nn(a.data_ptr(), b.data_ptr(), c.data_ptr(), offs.data_ptr(), g, rows, n, k,
                                          _lib.dt(a), ws, ws_bytes, st.cuda_stream))
    return c


def grouped_gemm_tn(a, b, offs, out=None, accumulate=False, stream=None):
    """c[g] (+)= a[rows_g].T @ b[rows_g] ; a [R, M], b [R, N] -> c [G, M, N]."""
    lib = _lib.load()
    g = offs.numel() - 1
    m, n = a.shape[1], b.shape[1]
    assert a.is_contiguous() and b.is_contiguous() and a.shape[0] == b.shape[0]
    st = stream or torch.cuda.current_stream()
    with torch.cuda.stream(st):
        if out is None:
            assert not accumulate
            out = torch.empty((g, m, n), dtype=a.dtype, device=a.device)
        _lib.check(lib.dh_grouped_gemm_tn(a.data_ptr(), b.data_ptr(), out.data_ptr(), offs.data_ptr(), g,
                                          a.shape[0], m, n, int(accumulate), _lib.dt(a), st.cuda_stream))
    return out


def expert_ffn_fwd(xp, w1, w2, offs, stream=None, profiling=False):
    """SwiGLU FFN of the local experts on permuted rows.  xp [R, H]; w1 [G, 2F, H] (gate |
    up); w2 [G, H, F]; offs int32 [G + 1] (a slice of MoEPlan.expert_offsets).
    Returns (y [R, H], (h, a) saved for backward, ms)."""
    from .swiglu import swiglu
    el: list = []
    with on_stream(stream, profiling, el) as st:
        h = grouped_gemm_nt(xp, w1, offs, stream=st)
        a, _ = swiglu(h, st)
        y = grouped_gemm_nt(a, w2, offs, stream=st)
    return y, (h, a), el[0]


def expert_ffn_bwd(dy, xp, w1, w2, offs, saved, dw1=None, dw2=None, stream=None, profiling=False):
    """Backward of expert_ffn_fwd.  Returns (dxp, dw1, dw2, ms); dw1/dw2 are accumulated
    into when given (the reference accumulates weight gradients into main_grad,
    dhellam/core/dstb.py:547-592)."""
    from .swiglu import swiglu_back
    h, a = saved
    el: list = []
    with on_stream(stream, profiling, el) as st:
        # data gradients: against the resident transposes of the expert weights where the caller keeps them
        # (``_Clib.keep_transposed``): the same products in the forward's layout, which the grouped kernel runs faster
        w2t, w1t = transposed_of(w2), transposed_of(w1)
        da = grouped_gemm_nt(dy, w2t, offs, stream=st) if w2t is not None else grouped_gemm_nn(dy, w2, offs, stream=st)   # [R, F] = dy @ w2[g]
        dw2 = grouped_gemm_tn(dy, a, offs, out=dw2, accumulate=dw2 is not None, stream=st)   # [G, H, F]
        dh, _ = swiglu_back(da, h, None, st)
        dxp = grouped_gemm_nt(dh, w1t, offs, stream=st) if w1t is not None else grouped_gemm_nn(dh, w1, offs, stream=st)   # [R, H] = dh @ w1[g]
        dw1 = grouped_gemm_tn(dh, xp, offs, out=dw1, accumulate=dw1 is not None, stream=st)  # [G, 2F, H]
        with torch.cuda.stream(st):
            _note_read(w2)
            _note_read(w1)
    return dxp, dw1, dw2, el[0]
