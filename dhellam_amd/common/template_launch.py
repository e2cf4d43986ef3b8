"""Stream/event launch templates: dhellam/common/template_launch.py:4-34."""
import torch


def _run(fn, stream, profiling):
    if stream is None:
        stream = torch.cuda.current_stream()
    elapsed = 0
    with torch.cuda.stream(stream):
        if profiling:
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record()
            out = fn()
            end.record()
            end.synchronize()
            elapsed = start.elapsed_time(end)
        else:
            out = fn()
    return out, elapsed


def template_fwd(fwd_func, inputs, stream, profiling):
    outputs, ms = _run(lambda: fwd_func(inputs), stream, profiling)
    return [inputs, outputs], ms


def template_bwd(bwd_func, ctx, grad_outputs, stream, profiling):
    return _run(lambda: bwd_func(ctx, grad_outputs), stream, profiling)
