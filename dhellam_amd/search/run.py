"""Profile, search and execute: the three stages of search/search.sh:163-183 on one GPU.

    python -m dhellam_amd.search.run [--out-dir DIR] [--seq 4096] [--repeat 5] [--top-k 6] [--steps 20]

1. profiler (search/profiler.py): time every candidate (forward group, backward group) pair -> ``op_profile_num.txt``;
2. search (search/search.py): the DP over those records, the ``--top-k`` cheapest plans -> ``candidates/*.json``,
   the cheapest also as ``best_result.json`` (the reference's name for the DP optimum);
3. execute (search/execute.py): replay every candidate and the built-in plan against the serial schedule, print
   ``sequence time / schedule time / speedup`` per candidate, write the measured winner to ``best.json`` and the
   table to ``execute_report.json``.

``bench.py`` runs the plan in ``dhellam_amd/search/config/best.json`` (the default ``--out-dir``) when there is one.
"""
from __future__ import annotations

import argparse
import json
import os
import time

import torch

from ..core.layer import LayerRunner, llama70b_tp8_shard, make_microbatch, make_weights
from .execute import BUILTIN, execute
from .op_table import operator_list_prune
from .profiler import profile_pairs
from .search import parse_op_file, plan_to_json, search_candidates_with_parking, unpaired_cost

CONFIG_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config")


def search_and_execute(cfg, weights, mbs, out_dir, repeat=5, top_k=6, steps=20, mode="device", log=print) -> dict:
    """All three stages; returns the execute report (also written to ``out_dir``)."""
    os.makedirs(os.path.join(out_dir, "candidates"), exist_ok=True)
    runner = LayerRunner(cfg, weights)
    prof_path = os.path.join(out_dir, "op_profile_num.txt")
    if os.path.exists(prof_path):
        os.remove(prof_path)
    t0 = time.perf_counter()
    profile_pairs(runner, mbs[0], prof_path, repeat=repeat, mode=mode)
    log(f"profiling took {time.perf_counter() - t0:.1f} s ({mode} timing)")
    prof = parse_op_file(prof_path)
    (_, _, fwd), (_, _, bwd) = operator_list_prune(cfg.context_parallel_size)
    fwd_alone, bwd_alone = unpaired_cost(prof, fwd, bwd)
    found = search_candidates_with_parking(prof, fwd, bwd, k=top_k)
    bwd_order = [x for g in bwd for x in g]
    candidates = []
    for rank, (cost, blocks, alias) in enumerate(found):
        plan = plan_to_json(blocks, alias=alias, bwd_order=bwd_order)
        name = f"dp_rank{rank}"
        with open(os.path.join(out_dir, "candidates", name + ".json"), "w") as f:
            json.dump(plan, f, indent=4)
        if rank == 0:
            with open(os.path.join(out_dir, "best_result.json"), "w") as f:
                json.dump(plan, f, indent=4)
        candidates.append({"name": name, "plan": plan, "paired_ms": cost})
        log(f"{name}: predicted paired phase {cost:.3f} ms (forward alone {fwd_alone:.3f} + backward alone "
            f"{bwd_alone:.3f} = {fwd_alone + bwd_alone:.3f}); deferred weight gradients: {sorted(alias.values())}")
    candidates.append({"name": BUILTIN, "plan": None})
    report = execute(cfg, weights, mbs, candidates, out_dir, steps=steps, fwd_alone_ms=fwd_alone,
                     bwd_alone_ms=bwd_alone, log=log)
    report["profile"] = {"timing": mode, "repeat": repeat, "forward_alone_ms": round(fwd_alone, 4),
                         "backward_alone_ms": round(bwd_alone, 4)}
    with open(os.path.join(out_dir, "execute_report.json"), "w") as f:
        json.dump(report, f, indent=1)
    b = report["best"]
    log(f"best: {b['name']} ({'lockstep' if b['lockstep_blocks'] else 'free-running'}) {b['ms']:.3f} ms, "
        f"speedup over the serial schedule {report['speedup_over_serial']:.4f} -> {os.path.join(out_dir, 'best.json')}")
    return report


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out-dir", default=CONFIG_DIR)
    ap.add_argument("--seq", type=int, default=4096)
    ap.add_argument("--repeat", type=int, default=5)
    ap.add_argument("--micro-batches", type=int, default=4)
    ap.add_argument("--top-k", type=int, default=6)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--timing", choices=("device", "reference"), default="device")
    args = ap.parse_args()
    cfg = llama70b_tp8_shard(seq_length=args.seq)
    w = make_weights(cfg, 0, gen_device="cuda")
    mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(args.micro_batches)]
    search_and_execute(cfg, w, mbs, args.out_dir, args.repeat, args.top_k, args.steps, args.timing,
                       log=lambda m: print(m, flush=True))


if __name__ == "__main__":
    main()
