"""The execute stage of the plan search: replay every candidate plan, keep the one that measures best.

Counterpart of search/execute.py:30-116: the reference walks every candidate JSON under ``config/dhellam-cp*/``,
times the serial schedule once (``fwd_only`` then ``bwd_only``, 20 repetitions, :63-75), times each candidate's
paired blocks (20 repetitions, :79-96), prints ``sequence time / schedule time / speedup`` per candidate and copies
the winner to ``config/best.json`` (:103-108).  Here a candidate is a plan dict (the k best of the DP plus the
built-in plan, so the emitted plan is never slower than what the runtime does without one); each is replayed through
``LayerRunner`` as a whole step of several micro-batches, free-running and with the strands entering every block
together (``lockstep_blocks``, the mode the DP's additive cost model describes); the winner is written to
``best.json`` next to a report that holds predicted and measured times of every candidate.
"""
from __future__ import annotations

import dataclasses
import json
import os
import time
from typing import Dict, List, Optional, Sequence

import torch

from ..core.dstb import DEFAULT_PLAN
from ..core.layer import LayerRunner

BUILTIN = "builtin"


def builtin_plan() -> dict:
    """The built-in paired / forward-only / backward-only plans (dhellam/core/dstb.py:1043-1129) as a plan dict."""
    return json.loads(json.dumps(DEFAULT_PLAN))


def _time_steps(fn, mbs, steps: int, warmup: int) -> float:
    for _ in range(warmup):
        fn(mbs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn(mbs)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def replay(cfg, weights, mbs, plan, steps: int = 20, warmup: int = 3, lockstep: bool = False) -> float:
    """ms per step of ``len(mbs)`` micro-batches under the double-strand schedule of ``plan`` (a dict, a path, or
    None for the built-in plan)."""
    runner = LayerRunner(dataclasses.replace(cfg, lockstep_blocks=bool(lockstep)), weights, plan=plan)
    return _time_steps(runner.run_double_strand, mbs, steps, warmup)


def replay_serial(cfg, weights, mbs, plan=None, steps: int = 20, warmup: int = 3) -> float:
    """ms per step of the serial schedule (one stream, ``fwd_only`` then ``bwd_only`` per micro-batch)."""
    return _time_steps(LayerRunner(cfg, weights, plan=plan).run_serial, mbs, steps, warmup)


def predicted_step_ms(paired_ms: float, fwd_alone_ms: float, bwd_alone_ms: float, n_microbatches: int) -> float:
    """What the DP's cost model says a step takes: the first forward and the last backward on their own and
    ``n - 1`` paired phases in between."""
    return fwd_alone_ms + max(0, n_microbatches - 1) * paired_ms + bwd_alone_ms


def execute(cfg, weights, mbs, candidates: Sequence[dict], out_dir: Optional[str] = None, steps: int = 20,
            warmup: int = 3, fwd_alone_ms: Optional[float] = None, bwd_alone_ms: Optional[float] = None,
            log=print) -> dict:
    """Replays ``candidates`` -- dicts {"name", "plan" (dict; None = built-in), "paired_ms" (the DP's cost of one
    paired phase, optional)} -- and returns the report: per candidate the measured step time free-running and in
    lockstep and the model's prediction; the serial time; the winner (smallest measured time over both modes,
    the built-in plan winning ties).  With ``out_dir`` the winner's plan goes to ``best.json`` there and the report
    to ``execute_report.json``."""
    cands = list(candidates)
    if not any(c["plan"] is None or c["name"] == BUILTIN for c in cands):
        cands.append({"name": BUILTIN, "plan": None})
    serial = replay_serial(cfg, weights, mbs, None, steps, warmup)
    n = len(mbs)
    rows: List[Dict] = []
    for i, c in enumerate(cands):
        free = replay(cfg, weights, mbs, c["plan"], steps, warmup, lockstep=False)
        lock = replay(cfg, weights, mbs, c["plan"], steps, warmup, lockstep=True)
        row = {"name": c["name"], "free_running_ms": round(free, 4), "lockstep_ms": round(lock, 4)}
        if c.get("paired_ms") is not None and fwd_alone_ms is not None and bwd_alone_ms is not None:
            pred = predicted_step_ms(c["paired_ms"], fwd_alone_ms, bwd_alone_ms, n)
            row["predicted_lockstep_ms"] = round(pred, 4)
            row["predicted_over_measured_lockstep"] = round(pred / lock, 4)
        rows.append(row)
        log(f"[{i + 1}/{len(cands)}] {c['name']}: sequence time {serial:.3f} ms  schedule time {free:.3f} ms "
            f"(lockstep {lock:.3f})  speedup {serial / min(free, lock):.4f}"
            + (f"  predicted lockstep {row['predicted_lockstep_ms']:.3f}" if "predicted_lockstep_ms" in row else ""))
    # the built-in plan wins ties: a searched plan must EARN its place (timer noise is a few tenths of a percent)
    order = sorted(range(len(rows)), key=lambda i: (min(rows[i]["free_running_ms"], rows[i]["lockstep_ms"]),
                                                    rows[i]["name"] != BUILTIN))
    w = order[0]
    win = rows[w]
    best = {"name": win["name"], "lockstep_blocks": win["lockstep_ms"] < win["free_running_ms"],
            "ms": min(win["free_running_ms"], win["lockstep_ms"])}
    report = {"micro_batches": n, "steps": steps, "serial_ms": round(serial, 4), "candidates": rows, "best": best,
              "speedup_over_serial": round(serial / best["ms"], 4)}
    if out_dir:
        os.makedirs(out_dir, exist_ok=True)
        plan = cands[w]["plan"] if cands[w]["plan"] is not None else builtin_plan()
        plan = json.load(open(plan)) if isinstance(plan, str) else plan
        with open(os.path.join(out_dir, "best.json"), "w") as f:
            json.dump(plan, f, indent=4)
        with open(os.path.join(out_dir, "execute_report.json"), "w") as f:
            json.dump(report, f, indent=1)
    return report
