"""SwiGLU forward/backward: dhellam/operators/swiglu.py:28-62.

``y`` has the gate in the first half of the last dim and the up projection in
the second half (swiglu.py:15).
"""
from __future__ import annotations

import torch

from .. import _lib
from ._util import on_stream


def _transposable(rows, f, *tensors) -> bool:
    """Shapes, types and alignment that the kernels with a transposed second output take."""
    return (rows > 0 and f > 0 and rows % 8 == 0 and f % 8 == 0 and rows < 64 * 65535
            and all(t.dtype in (torch.bfloat16, torch.float16) and t.dtype == tensors[0].dtype
                    and t.data_ptr() % 16 == 0 for t in tensors))


def swiglu(y, stream=None, profiling=False, with_transposed=False):
    """``with_transposed``: the kernel also writes the result transposed ([f, rows], for the weight-gradient product
    of the projection behind the activation) and hangs it on the returned tensor, where ``_Clib.wgrad_gemm`` finds
    it; ignored for shapes or types the kernel does not take."""
    assert y.is_cuda and y.is_contiguous() and y.shape[-1] % 2 == 0
    lib = _lib.load()
    f = y.shape[-1] // 2
    rows = y.numel() // (2 * f) if f else 0
    el: list = []
    with on_stream(stream, profiling, el) as st:
        out = torch.empty(*y.shape[:-1], f, dtype=y.dtype, device=y.device)
        if with_transposed and _transposable(rows, f, y, out):
            ot = torch.empty((f, rows), dtype=y.dtype, device=y.device)
            _lib.check(lib.dh_swiglu_fwd_t(y.data_ptr(), out.data_ptr(), ot.data_ptr(), rows, f, _lib.dt(y),
                                           st.cuda_stream))
            out._dh_rows_transposed = (out._version, ot)    # valid while nothing has written ``out`` since
        else:
            _lib.check(lib.dh_swiglu_fwd(y.data_ptr(), out.data_ptr(), rows, f, _lib.dt(y), st.cuda_stream))
    return out, el[0]


def swiglu_back(g, y, o=None, stream=None, profiling=False, with_transposed=False):
    """``o`` (optional) receives the result; the reference allocates it but its kernel
    ignores it (swiglu.py:48-55).  ``with_transposed``: the kernel also writes the result transposed
    ([2f, rows], for the weight-gradient product of the projection in front of the activation) and hangs it on the
    returned tensor, where ``_Clib.wgrad_gemm`` finds it; ignored for shapes or types the kernel does not take."""
    assert y.is_cuda and y.is_contiguous() and g.is_contiguous() and y.shape[-1] % 2 == 0
    lib = _lib.load()
    f = y.shape[-1] // 2
    rows = y.numel() // (2 * f) if f else 0
    assert g.numel() == rows * f, "grad shape does not match swiglu input"
    el: list = []
    with on_stream(stream, profiling, el) as st:
        if o is None:
            o = torch.empty_like(y)
        assert o.is_contiguous() and o.shape == y.shape
        if with_transposed and _transposable(rows, f, y, g, o):
            ot = torch.empty((2 * f, rows), dtype=y.dtype, device=y.device)
            _lib.check(lib.dh_swiglu_bwd_t(g.data_ptr(), y.data_ptr(), o.data_ptr(), ot.data_ptr(), rows, f, _lib.dt(y),
                                           st.cuda_stream))
            o._dh_rows_transposed = (o._version, ot)    # valid while nothing has written ``o`` since
        else:
            _lib.mark_written(o)            # a reused ``o`` may carry the transposed twin of an earlier call
            _lib.check(lib.dh_swiglu_bwd(g.data_ptr(), y.data_ptr(), o.data_ptr(), rows, f, _lib.dt(y), st.cuda_stream))
    return o, el[0]
