"""Norm forward/backward with the reference's wrapper signatures.

Mirrors dhellam/operators/layernorm.py:6-45 (``pylayernorm_fwd``) and :47-91
(``pylayernorm_bwd``).  ``ln_bias=None`` selects RMSNorm (returned ``mu`` is
None); a bias selects LayerNorm.  ``fwd_sm_margin`` / ``bwd_sm_margin`` are
accepted and ignored (every reference call site passes 0, dstb.py:70,77,388).
"""
from __future__ import annotations

import torch

from .. import _lib
from ._util import on_stream

_workspaces: dict = {}


def _workspace(nbytes: int, device, stream) -> torch.Tensor:
    """fp32 scratch for the dgamma partial rows, cached per (device, stream)."""
    key = (device, stream.cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() * 4 < nbytes:
        ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=device)
        _workspaces[key] = ws
    return ws


def pylayernorm_fwd(inp, ln_weight, ln_bias, eps, fwd_sm_margin, zero_centered_gamma, stream, profiling=False,
                    residual=None, sum_out=None, ln_out=None):
    """Returns (ln_out, mu, rsigma, ms).  Extension over the reference signature: with ``residual`` the row that
    is normalised is ``inp + residual``, which is also stored in ``sum_out`` (default: a new tensor, returned
    as a fifth value) -- the reference's bda op and the norm after it (dstb.py:273-277, 73-78) in one pass.
    ``ln_out``: a contiguous tensor of the input's size to write the result into (e.g. this rank's rows of the
    buffer a sequence-parallel all-gather fills) instead of a new one."""
    in_features = ln_weight.numel()
    assert inp.is_cuda, "dhellam needs a GPU."
    assert inp.shape[-1] == in_features, "LayerNorm not possible"
    assert inp.is_contiguous() and ln_weight.is_contiguous()
    lib = _lib.load()
    inputmat = inp.view((-1, in_features))
    rows = inputmat.shape[0]
    el: list = []
    with on_stream(stream, profiling, el) as st:
        if ln_out is None:
            ln_out = torch.empty_like(inputmat)
        else:
            assert ln_out.is_contiguous() and ln_out.numel() == inputmat.numel() and ln_out.dtype == inputmat.dtype
            _lib.mark_written(ln_out)
        rsigma = torch.empty(rows, dtype=torch.float32, device=inp.device)
        mu = torch.empty(rows, dtype=torch.float32, device=inp.device) if ln_bias is not None else None
        if residual is None:
            _lib.check(lib.dh_norm_fwd(inputmat.data_ptr(), ln_weight.data_ptr(), _lib.ptr(ln_bias), ln_out.data_ptr(),
                                       _lib.ptr(mu), rsigma.data_ptr(), rows, in_features, float(eps),
                                       int(bool(zero_centered_gamma)), _lib.dt(inp), st.cuda_stream))
        else:
            assert residual.is_contiguous() and residual.numel() == inp.numel() and residual.dtype == inp.dtype
            if sum_out is None:
                sum_out = torch.empty_like(residual)
            assert sum_out.is_contiguous() and sum_out.numel() == inp.numel() and sum_out.dtype == inp.dtype
            _lib.check(lib.dh_add_norm_fwd(inputmat.data_ptr(), residual.data_ptr(), sum_out.data_ptr(),
                                           ln_weight.data_ptr(), _lib.ptr(ln_bias), ln_out.data_ptr(), _lib.ptr(mu),
                                           rsigma.data_ptr(), rows, in_features, float(eps),
                                           int(bool(zero_centered_gamma)), _lib.dt(inp), st.cuda_stream))
    if residual is not None:
        return ln_out.view_as(inp), mu, rsigma, el[0], sum_out
    return ln_out.view_as(inp), mu, rsigma, el[0]


def pylayernorm_bwd(d_ln_out, inp, mu, rsigma, ln_weight, bwd_sm_margin, zero_centered_gamma, stream,
                    profiling=False, add_to_dgrad=None, dgamma_out=None, dbeta_out=None, dgrad_out=None):
    """Returns (dinp, dgamma, dbeta, ms).

    Extensions over the reference signature (all optional): ``add_to_dgrad`` is
    added to dinp inside the kernel (the residual-branch gradient the reference
    adds afterwards, dstb.py:391,401); ``dgamma_out`` / ``dbeta_out`` are
    accumulated into in place (the reference's ``main_grad.add_``, dstb.py:392-393);
    ``dgrad_out`` is a contiguous tensor of the input's size that receives dinp instead of a new one.
    """
    in_features = ln_weight.numel()
    assert inp.is_cuda, "dhellam needs a GPU."
    assert inp.shape[-1] == in_features, "LayerNorm not possible"
    lib = _lib.load()
    inputmat = inp.view((-1, in_features))
    d_ln_out = d_ln_out.view((-1, in_features))
    assert inputmat.is_contiguous() and d_ln_out.is_contiguous()
    rows = inputmat.shape[0]
    el: list = []
    with on_stream(stream, profiling, el) as st:
        if dgrad_out is None:
            dinp = torch.empty_like(inputmat)
        else:
            assert dgrad_out.is_contiguous() and dgrad_out.numel() == inputmat.numel() and dgrad_out.dtype == inputmat.dtype
            _lib.mark_written(dgrad_out)
            dinp = dgrad_out.view(inputmat.shape)
        accumulate = dgamma_out is not None
        assert not accumulate or dgamma_out.dtype == ln_weight.dtype, "dgamma_out must have the weight's dtype"
        assert dbeta_out is None or dbeta_out.dtype == ln_weight.dtype, "dbeta_out must have the weight's dtype"
        dgamma = dgamma_out if accumulate else torch.empty_like(ln_weight)
        if mu is not None:
            dbeta = dbeta_out if dbeta_out is not None else torch.empty_like(ln_weight)
            assert (dbeta_out is not None) == accumulate, "pass both or neither of dgamma_out/dbeta_out"
        else:
            dbeta = None
        ws = _workspace(lib.dh_norm_bwd_workspace_bytes(rows, in_features), inp.device, st)
        add = add_to_dgrad.view((-1, in_features)) if add_to_dgrad is not None else None
        _lib.check(lib.dh_norm_bwd(d_ln_out.data_ptr(), inputmat.data_ptr(), _lib.ptr(mu), rsigma.data_ptr(),
                                   ln_weight.data_ptr(), _lib.ptr(add), dinp.data_ptr(), dgamma.data_ptr(),
                                   _lib.ptr(dbeta), ws.data_ptr(), ws.numel() * ws.element_size(), rows, in_features,
                                   int(bool(zero_centered_gamma)), int(accumulate), _lib.dt(inp), st.cuda_stream))
    return dinp.view_as(inp), dgamma, dbeta, el[0]
