"""Shared plumbing of the operator wrappers: the (stream, profiling) convention.

Every reference operator takes ``stream`` (None = current stream), runs its body
under ``torch.cuda.stream(stream)`` and returns a trailing elapsed-time value that
is 0 unless ``profiling`` (dhellam/operators/swiglu.py:28-43,
dhellam/common/template_launch.py:4-19).  Elapsed time is always milliseconds
here (the reference's norm wrapper returns seconds, layernorm.py:36-40).
"""
from __future__ import annotations

import contextlib

import torch


@contextlib.contextmanager
def on_stream(stream, profiling: bool, elapsed: list):
    """Run the body on ``stream``; with ``profiling`` bracket it with events and
    append the elapsed milliseconds to ``elapsed`` (else append 0)."""
    if stream is None:
        stream = torch.cuda.current_stream()
    with torch.cuda.stream(stream):
        if profiling:
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record()
            yield stream
            end.record()
            end.synchronize()
            elapsed.append(start.elapsed_time(end))
        else:
            yield stream
            elapsed.append(0)
