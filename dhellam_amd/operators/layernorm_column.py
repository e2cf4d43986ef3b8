"""Dense projection GEMMs with the reference's wrapper signatures.

Mirrors dhellam/operators/layernorm_column.py:7-62 (``gemm_fwd``), :209-263
(``dgrad_bwd``) and :265-323 (``wgrad_bwd``).  Weights are stored [out, in];
the layout letters are the reference's: "TN" computes input @ weight.T, "NN"
grad @ weight, "NT" grad.T @ input.  Dense GEMM is a library call on this path:
``dh_gemm`` of the C ABI (hipBLASLt) whichever way it is asked for.  ``is_matmul=True``
(what every scheduler call site of the reference selects, dhellam/core/dstb.py:84-106,
300-340) takes inputs with leading dimensions, as ``torch.matmul`` does there, and falls back
to ``torch.matmul`` only for operands ``dh_gemm`` does not take (strided views, mixed types);
``is_matmul=False`` is ``_Clib.pygemm`` with its contiguous 2-D operands.
Output dtype follows the inputs (the reference hard-codes fp16).  Elapsed time
is in milliseconds, measured with events on the op's stream.
"""
from __future__ import annotations

from typing import Optional

import torch

from .._Clib import _note_read, dense_gemm, dense_ok, dgrad_gemm, transposed_of
from .._Clib import pygemm as gemm
from .._Clib import wgrad_gemm
from ._util import on_stream


def gemm_fwd(args, input: torch.Tensor, weight: torch.Tensor, output: Optional[torch.Tensor] = None,
             layout: str = "TN", profiling: bool = False, math_sm_count: int = 0, is_matmul: bool = False,
             stream=None):
    transa = layout[0] == "T"
    transb = layout[1] == "T"
    el: list = []
    with on_stream(stream, profiling, el):
        if is_matmul:
            x2 = input.reshape(-1, input.shape[-1]) if input.is_contiguous() else input
            if (transa and not transb and dense_ok(weight, x2) and weight.dtype == input.dtype
                    and (output is None or (output.is_contiguous() and output.dtype == input.dtype))):
                if output is None:
                    output = torch.empty(*input.shape[:-1], weight.shape[0], dtype=input.dtype, device=input.device)
                dense_gemm(weight, x2, output.view(-1, weight.shape[0]), True, False, False)
            else:
                w = weight.t() if transa else weight
                x = input.t() if transb else input
                output = torch.matmul(x, w) if output is None else torch.matmul(x, w, out=output)
        else:
            if output is None:
                output = torch.empty(input.shape[1] if transb else input.shape[0],
                                     weight.shape[0] if transa else weight.shape[1], dtype=input.dtype,
                                     device=input.device)
            gemm(weight, input, output, None, 0, transa, transb, False, math_sm_count, False)
    return output, el[0]


def gemm_fwd_event(args, input: torch.Tensor, weight: torch.Tensor, output: Optional[torch.Tensor] = None,
                   layout: str = "TN", profiling: bool = False, math_sm_count: int = 0, is_matmul: bool = False):
    """layernorm_column.py:64-119: ``gemm_fwd`` on the current stream (the reference's variant without a
    ``stream`` argument, timed with events like every operator here)."""
    return gemm_fwd(args, input, weight, output, layout, profiling, math_sm_count, is_matmul, None)


def dgrad_bwd(args, input_grad: torch.Tensor, weight: torch.Tensor, dgrad_output: Optional[torch.Tensor],
              layout: str = "NN", profiling: bool = False, math_sm_count: int = 0, is_matmul: bool = False,
              stream=None):
    transa = layout[0] == "T"
    transb = layout[1] == "T"
    el: list = []
    with on_stream(stream, profiling, el):
        if dgrad_output is None:
            dgrad_output = torch.empty(input_grad.shape[1] if transb else input_grad.shape[0],
                                       weight.shape[0] if transa else weight.shape[1], dtype=input_grad.dtype,
                                       device=input_grad.device)
        if is_matmul:
            if (not transa and not transb and dense_ok(weight, input_grad, dgrad_output)
                    and weight.dtype == input_grad.dtype == dgrad_output.dtype):
                dgrad_gemm(input_grad, weight, dgrad_output)
            else:
                w = weight.t() if transa else weight
                g = input_grad.t() if transb else input_grad
                torch.matmul(g, w, out=dgrad_output)
        else:
            wt = transposed_of(weight) if not (transa or transb) else None
            if wt is not None and wt.dtype == input_grad.dtype:      # same product in the forward's layout
                gemm(wt, input_grad, dgrad_output, None, 0, True, False, False, math_sm_count, False)
                _note_read(weight)
            else:
                gemm(weight, input_grad, dgrad_output, None, 0, transa, transb, False, math_sm_count, False)
    return dgrad_output, el[0]


def wgrad_bwd(args, input_grad: torch.Tensor, input_data: torch.Tensor, wgrad_output: Optional[torch.Tensor],
              grad_accumulate: bool = False, layout: str = "NT", profiling: bool = False, math_sm_count: int = 0,
              is_matmul: bool = False, stream=None):
    """wgrad [out, in] = input_grad.T @ input_data.  As in the reference's matmul path
    (layernorm_column.py:289-292) a given ``wgrad_output`` is ACCUMULATED into."""
    transa = layout[0] == "T"
    transb = layout[1] == "T"
    el: list = []
    with on_stream(stream, profiling, el):
        if is_matmul:
            fresh = wgrad_output is None
            dt = input_grad.dtype
            if (transb and not transa and dense_ok(input_grad, input_data) and dt == input_data.dtype
                    and (fresh or (dense_ok(wgrad_output) and wgrad_output.dtype in (dt, torch.float32)))):
                if fresh:
                    wgrad_output = torch.empty(input_grad.shape[1], input_data.shape[1], dtype=dt, device=input_grad.device)
                wgrad_gemm(input_grad, input_data, wgrad_output, not fresh)
            else:
                d = input_data.t() if transa else input_data
                g = input_grad.t() if transb else input_grad
                if fresh:
                    wgrad_output = torch.matmul(g, d)
                elif wgrad_output.dtype == g.dtype:
                    wgrad_output.addmm_(g, d)
                else:  # fp32 main_grad with 16-bit operands
                    wgrad_output.add_(torch.matmul(g, d))
        else:
            if wgrad_output is None:
                wgrad_output = torch.empty(input_grad.shape[1] if transb else input_grad.shape[0],
                                           input_data.shape[0] if transa else input_data.shape[1],
                                           dtype=input_grad.dtype, device=input_grad.device)
                grad_accumulate = False
            gemm(input_data, input_grad, wgrad_output, None, 0, transa, transb, grad_accumulate, math_sm_count, False)
    return wgrad_output, el[0]


def gemm_bwd(args, input_grad, input_data, weight, dgrad_output=None, wgrad_output=None, grad_accumulate=False,
             profiling=False, math_sm_count=0, is_matmul=True, stream=None):
    """dgrad then wgrad of one projection (layernorm_column.py:121-207).
    Returns (dgrad, wgrad, dgrad_ms, wgrad_ms)."""
    dgrad_output, t1 = dgrad_bwd(args, input_grad, weight, dgrad_output, "NN", profiling, math_sm_count, is_matmul, stream)
    wgrad_output, t2 = wgrad_bwd(args, input_grad, input_data, wgrad_output, grad_accumulate, "NT", profiling,
                                 math_sm_count, is_matmul, stream)
    return dgrad_output, wgrad_output, t1, t2


gemm_fwd_event = gemm_fwd  # the reference's event-timed twin (layernorm_column.py:64-119); timing is always by event here
