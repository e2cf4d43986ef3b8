"""Timing harnesses: dhellam/common/benchmark.py.

``benchmark_ms_ops`` is the protocol the plan search is built on (benchmark.py:31-79):
wall-clock time of launching one list of prepared ops on stream s1 and another on s2,
bracketed by device synchronisation, repeated ``repeat`` times, with the 20 % tails
trimmed only when there are more than 10 samples.
"""
import time

import torch


def benchmark(repeat, fn, *args, **kwargs):
    """Mean wall-clock ms of fn(*args) with a device sync on both sides (benchmark.py:4-14)."""
    times = []
    for _ in range(repeat):
        torch.cuda.synchronize()
        start = time.perf_counter()
        fn(*args, **kwargs)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - start) * 1000)
    return sum(times) / repeat


def benchmark_ms(repeat, s1, s2, fn1, fn2, *args):
    """Mean ms of ``repeat`` rounds of one prepared op on s1 and one on s2 (benchmark.py:17-29); a factory is
    ``fn(*args) -> (call_args, callable)``."""
    a1, k1 = fn1(*args)
    a2, k2 = fn2(*args)
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(repeat):
        with torch.cuda.stream(s1):
            k1(*a1)
        with torch.cuda.stream(s2):
            k2(*a2)
    torch.cuda.synchronize()
    return (time.perf_counter() - start) / repeat * 1000


def trimmed_mean(samples):
    """Mean after dropping the lowest and highest 20 %, only when more than 10 samples."""
    s = sorted(samples)
    drop = int(len(s) * 0.2)
    if drop > 0 and len(s) > 10:
        s = s[drop:-drop]
    return sum(s) / len(s) if s else 0.0


def benchmark_ms_ops(repeat, s1, s2, fn1, fn2, fn3, *args):
    """fn1 / fn2: lists of factories ``op(*args, stream) -> (call_args, callable)``; the
    callables of fn1 are launched (on s1), then those of fn2 (on s2).  fn3 (the reference's
    communication op) must be None on one GPU.  Returns the trimmed mean in ms."""
    if fn3 is not None:
        raise ValueError("communication ops are not part of the single-GPU path")
    l1 = [op(*args, s1) for op in (fn1 or [])]
    l2 = [op(*args, s2) for op in (fn2 or [])]
    samples = []
    for _ in range(repeat):
        torch.cuda.synchronize()
        start = time.perf_counter()
        for call_args, fn in l1:
            fn(*call_args)
        for call_args, fn in l2:
            fn(*call_args)
        torch.cuda.synchronize()
        samples.append(time.perf_counter() - start)
    return trimmed_mean(samples) * 1000
