"""Bias-dropout-add slot, run as a plain residual add: dhellam/operators/bda.py:14-49.

The reference hard-codes dropout p = 0.1 (bda.py:5); here ``p`` is a parameter
and only p = 0 is implemented (the mask is all ones and never materialised
unless asked for).
"""
from __future__ import annotations

import torch

from .. import _lib
from ._util import on_stream


def bda_fwd(input, residual, stream=None, profiling=False, p: float = 0.0, return_mask: bool = False, out=None):
    """In place on ``input`` like the reference, unless ``out`` (same numel/dtype) is given.
    Returns (output, mask, ms); mask is None unless ``return_mask`` (then an int8 ones
    tensor)."""
    if p != 0.0:
        raise NotImplementedError("bda_fwd: only p = 0 (no dropout) is implemented")
    assert input.is_cuda and input.is_contiguous() and residual.is_contiguous()
    assert input.numel() == residual.numel() and input.dtype == residual.dtype
    lib = _lib.load()
    el: list = []
    with on_stream(stream, profiling, el) as st:
        dst = input if out is None else out
        assert dst.is_contiguous() and dst.numel() == input.numel() and dst.dtype == input.dtype
        _lib.check(lib.dh_residual_add(input.data_ptr(), residual.data_ptr(), dst.data_ptr(), input.numel(),
                                       _lib.dt(input), st.cuda_stream))
        mask = torch.ones_like(input, dtype=torch.int8) if return_mask else None
    return dst, mask, el[0]


def bda_bwd(dgrad, mask, output=None, stream=None, profiling=False):
    """Returns (dgrad_residual, dgrad_input, ms).  With p = 0 both branches receive
    ``dgrad`` itself; no kernel runs (``mask`` must be None or all ones)."""
    el: list = []
    with on_stream(stream, profiling, el):
        if output is not None:
            output.copy_(dgrad)
            dgrad_input = output
        else:
            dgrad_input = dgrad
    return dgrad, dgrad_input, el[0]
