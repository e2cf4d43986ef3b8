"""Stream/event launch templates: dhellam/common/template_launch.py:4-72."""
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


def template_fwd_new(fwd_func, *inputs, stream=None, profiling=False):
    """template_launch.py:36-52: run ``fwd_func(*inputs)`` on ``stream``; the context is
    [the inputs that need a gradient, the outputs]."""
    outputs, ms = _run(lambda: fwd_func(*inputs), stream, profiling)
    return [[each for each in inputs if isinstance(each, torch.Tensor) and each.requires_grad], outputs], ms


def template_bwd_new(ctx, grad_outputs, stream=None, profiling=False):
    """template_launch.py:54-72: autograd backward of a ``template_fwd_new`` context on ``stream``; returns
    the gradients of the recorded inputs."""
    def run():
        torch.autograd.backward(ctx[1], grad_tensors=grad_outputs, inputs=ctx[0] if ctx[0] else None)
        return [each.grad for each in ctx[0]]
    return _run(run, stream, profiling)
