"""Rotary position embedding on q and k (rotate-half).

The reference has no RoPE; these wrappers follow its operator convention and sit
where a Llama layer needs them: after the q/k/v split and before the attention
call (dhellam/core/dstb.py:122-126), and on dq/dk before the dq|dk|dv concat in
backward (:376-382).
"""
from __future__ import annotations

import torch

from .. import _lib
from ._util import on_stream

_inv_freq_cache: dict = {}


def rope_inv_freq(theta: float, d: int, device) -> torch.Tensor:
    """fp32 [d/2] table theta^(-2j/d), evaluated in double and rounded once."""
    key = (float(theta), int(d), str(device))
    t = _inv_freq_cache.get(key)
    if t is None:
        vals = [float(theta) ** (-2.0 * j / d) for j in range(d // 2)]
        t = torch.tensor(vals, dtype=torch.float64).to(torch.float32).to(device)
        _inv_freq_cache[key] = t
    return t


def _token_stride(t: torch.Tensor) -> int:
    assert t.dim() == 3 and t.stride(2) == 1 and t.stride(1) == t.shape[2], \
        "expected [tokens, heads, d] with contiguous heads"
    return t.stride(0)


def _rope(q, k, positions, theta, seq_len, backward, stream, profiling, inplace):
    assert q.is_cuda
    lib = _lib.load()
    d = q.shape[-1]
    inv = rope_inv_freq(theta, d, q.device)
    if positions is not None:
        assert positions.dtype == torch.int32 and positions.numel() == q.shape[0]
    el: list = []
    with on_stream(stream, profiling, el) as st:
        qo = q if inplace else torch.empty(q.shape, dtype=q.dtype, device=q.device)
        ko = None
        if k is not None:
            assert k.shape[0] == q.shape[0] and k.shape[-1] == d and k.dtype == q.dtype
            ko = k if inplace else torch.empty(k.shape, dtype=k.dtype, device=k.device)
        _lib.check(lib.dh_rope(q.data_ptr(), _lib.ptr(k), qo.data_ptr(), _lib.ptr(ko), inv.data_ptr(),
                               _lib.ptr(positions), q.shape[0], q.shape[1], k.shape[1] if k is not None else 0, d,
                               _token_stride(q), _token_stride(k) if k is not None else 0, _token_stride(qo),
                               _token_stride(ko) if ko is not None else 0, int(seq_len or 0), int(backward),
                               _lib.dt(q), st.cuda_stream))
    return qo, ko, el[0]


def rope_fwd(q, k, positions=None, theta=10000.0, seq_len=None, stream=None, profiling=False, inplace=False):
    """q [tokens, hq, d], k [tokens, hk, d] (views with a token stride are fine).
    positions: int32 [tokens], or None for pos = t % seq_len (t if seq_len is None).
    Returns (q_rot, k_rot, ms)."""
    return _rope(q, k, positions, theta, seq_len, False, stream, profiling, inplace)


def rope_bwd(dq, dk, positions=None, theta=10000.0, seq_len=None, stream=None, profiling=False, inplace=False):
    """Gradient of rope_fwd: the inverse rotation applied to dq, dk."""
    return _rope(dq, dk, positions, theta, seq_len, True, stream, profiling, inplace)
