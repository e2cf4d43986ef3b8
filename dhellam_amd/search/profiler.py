"""Single-GPU profiling pass: time every (forward group, backward group) pair on one stream
and on two streams.

Counterpart of search/profiler.py:20-65,142-180.  The reference builds each op's inputs
from random tensors in per-op factories (search/op_table.py:127-361); here one real
forward and backward of the layer is RECORDED (each op's input and the activation entries
it consumes), and an op is re-issued from that record -- shapes, strides and dtypes are the
ones the layer really uses.  Two timing protocols.  "reference": as in the reference, one warm-up launch
each for (s1,s2), (s1,s1), (s2,s2), then 5 serial and 5 two-stream repetitions of ``benchmark_ms_ops`` (host
clock, a device synchronisation around every repetition: right for a runtime that synchronises after every
block, dhellam/core/dstb.py:1266).  "device" (the default here): the time the pair takes ON THE GPU when the
launch queue is full, which is how this runtime executes a plan (nothing in ``exec`` waits for the device, so
launch latency is hidden behind earlier work): the repetitions are queued behind a delay kernel that lets the
host get ahead, separated by the same stream-to-stream event edges that ``lockstep_blocks`` puts between two
blocks, and timed with events on the stream.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import _lib
from ..common.benchmark import benchmark_ms_ops
from ..core import dstb
from ..core.layer import LayerRunner, fresh_activation_dict
from .op_table import ID_TO_NAME, OP_TABLE_IDX, PLAN_NAME, get_candidate_operator_groups
from .search import format_record


class _Recorder:
    """DCoperation look-alike that stores (input, activation snapshot) per op name."""

    def __init__(self):
        self.records: Dict[str, tuple] = {}

    def perform_operation(self, dcfunc, operation, config, weight, activation_dict, **kw):
        name = kw.get("name")
        snap = dict(activation_dict)
        out = dstb.DCoperation.perform_operation(dcfunc, operation, config, weight, activation_dict, **kw)
        self.records[name] = (operation, kw.get("output"), snap, weight)
        return out


def record_layer(runner: LayerRunner, mb: dict) -> Dict[str, tuple]:
    """Run one forward and one backward on one stream and record every op."""
    rec = _Recorder()
    s = runner.stream1
    s.wait_stream(torch.cuda.current_stream())
    act = fresh_activation_dict(mb)
    dstb.exec(runner.cfg, rec, runner.weights, None, mb["x"], None, runner.plan.fwd_only, s, s, None, act)
    dstb.exec(runner.cfg, rec, None, runner.weights, None, mb["dy"], runner.plan.bwd_only, s, s, act, None)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    return rec.records


def op_factory(records, cfg, op_id: int):
    """``factory(stream) -> (args, fn)`` re-issuing one recorded op (plus the stand-in comm op
    that feeds it is NOT included: its cost is a few microseconds and it is not a search variable)."""
    name = ID_TO_NAME[op_id]
    name = PLAN_NAME.get(name, name)
    operation, inp, snap, weight = records[name]

    def factory(stream):
        def fn():
            dstb.DCoperation.perform_operation(dstb.DCFunc, operation, cfg, weight, dict(snap), output=inp,
                                               stream=stream, name=name)
        return (), fn
    return factory


HOST_US_PER_OP = 150.0      # generous bound of what the host needs to queue one op (sizes the lead-in delay)


def _device_ms(fn1, fn2, sa, sb, repeat: int) -> float:
    """ms per repetition, on the device, of the ops of fn1 on ``sa`` and of fn2 on ``sb`` (``sa is sb``: one after
    the other on one stream).  Every repetition starts with both streams joined, like a block of a lockstep plan."""
    lib = _lib.load()
    l1 = [op(sa) for op in fn1]
    l2 = [op(sb) for op in fn2]
    two = sb.cuda_stream != sa.cuda_stream

    def join():
        if two:
            e1, e2 = torch.cuda.Event(), torch.cuda.Event()
            e1.record(sa)
            e2.record(sb)
            sa.wait_event(e2)
            sb.wait_event(e1)

    join()
    lead_ns = int((200.0 + HOST_US_PER_OP * repeat * (len(l1) + len(l2) + 2)) * 1e3)
    _lib.check(lib.dh_delay(lead_ns, sa.cuda_stream))          # the host queues everything below meanwhile
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(sa)
    for _ in range(repeat):
        join()
        for _, fn in l1:
            fn()
        for _, fn in l2:
            fn()
    join()
    end.record(sa)
    end.synchronize()
    return start.elapsed_time(end) / repeat


def time_pair(records, cfg, fwd_ids: List[int], bwd_ids: List[int], s1, s2, repeat: int = 5, mode: str = "device"):
    """(speedup, seq_time, para_time) of one pair; ``mode`` "reference" is the protocol of
    search/profiler.py:46-56, "device" times the pair on the GPU with the launch queue full (module docstring)."""
    fn1 = [op_factory(records, cfg, i) for i in fwd_ids]
    fn2 = [op_factory(records, cfg, i) for i in bwd_ids]
    if mode == "device":
        _device_ms(fn1, fn2, s1, s2, 1)                         # warm-up (first-use allocations, library plans)
        seq = _device_ms(fn1, fn2, s1, s1, repeat)
        par = _device_ms(fn1, fn2, s1, s2, repeat)
        return (seq / par if par > 0 else 1.0), seq, par
    if mode != "reference":
        raise ValueError(f"unknown timing mode {mode!r}")
    benchmark_ms_ops(1, s1, s2, fn1, fn2, None)
    benchmark_ms_ops(1, s1, s1, fn1, fn2, None)
    benchmark_ms_ops(1, s2, s2, fn1, fn2, None)
    seq = benchmark_ms_ops(repeat, s1, s1, fn1, fn2, None)
    par = benchmark_ms_ops(repeat, s1, s2, fn1, fn2, None)
    return (seq / par if par > 0 else 1.0), seq, par


def profile_pairs(runner: LayerRunner, mb: dict, out_path: Optional[str] = None, repeat: int = 5, progress=None,
                  mode: str = "device"):
    """Time every candidate pair; returns {(fwd ids, bwd ids): para_time ms} and, when
    ``out_path`` is given, appends the records to it in the op_profile_num.txt format."""
    records = record_layer(runner, mb)
    fwd_c, bwd_c = get_candidate_operator_groups(runner.cfg.context_parallel_size)
    s1, s2 = runner.stream1, runner.stream2
    prof = {}
    fp = open(out_path, "a") if out_path else None
    try:
        for fi, f in enumerate(fwd_c):
            for b in bwd_c:
                if not f and not b:
                    continue
                sp, seq, par = time_pair(records, runner.cfg, f, b, s1, s2, repeat, mode)
                prof[(tuple(f), tuple(b))] = par
                if fp:
                    fp.write(format_record(f, b, sp, seq, par))
            if progress:
                progress(fi + 1, len(fwd_c))
    finally:
        if fp:
            fp.close()
    return prof
