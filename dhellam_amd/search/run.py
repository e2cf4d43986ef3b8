"""Profile, search and validate a double-strand plan on one GPU.

    python -m dhellam_amd.search.run [--out-dir DIR] [--seq 4096] [--repeat 5]

The three stages of search/search.sh:163-183 (profiler, search, execute): time every
candidate (forward group, backward group) pair, run the DP, write
``op_profile_num.txt`` and ``best_result.json``, then replay the plan against the serial
schedule (search/execute.py:54-107) and print both times.
"""
from __future__ import annotations

import argparse
import json
import os
import time

import torch

from ..core.layer import LayerRunner, llama70b_tp8_shard, make_microbatch, make_weights
from .op_table import operator_list_prune
from .profiler import profile_pairs
from .search import dump_plan, parse_op_file, search_plan_with_parking


def validate(cfg, weights, mbs, plan_path, steps=10, warmup=3):
    """(serial ms, double-strand ms) per step of len(mbs) micro-batches."""
    runner = LayerRunner(cfg, weights, plan=plan_path)

    def timed(fn):
        for _ in range(warmup):
            fn(mbs)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn(mbs)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3
    return timed(runner.run_serial), timed(runner.run_double_strand)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out-dir", default="search_out")
    ap.add_argument("--seq", type=int, default=4096)
    ap.add_argument("--repeat", type=int, default=5)
    ap.add_argument("--micro-batches", type=int, default=4)
    args = ap.parse_args()
    os.makedirs(args.out_dir, exist_ok=True)
    cfg = llama70b_tp8_shard(seq_length=args.seq)
    w = make_weights(cfg, 0, gen_device="cuda")
    mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(args.micro_batches)]
    runner = LayerRunner(cfg, w)
    prof_path = os.path.join(args.out_dir, "op_profile_num.txt")
    if os.path.exists(prof_path):
        os.remove(prof_path)
    t0 = time.perf_counter()
    profile_pairs(runner, mbs[0], prof_path, repeat=args.repeat,
                  progress=lambda i, n: print(f"profiled forward group {i}/{n}", flush=True))
    print(f"profiling took {time.perf_counter() - t0:.1f} s", flush=True)
    prof = parse_op_file(prof_path)
    (_, _, fwd), (_, _, bwd) = operator_list_prune(cfg.context_parallel_size)
    cost, blocks, alias = search_plan_with_parking(prof, fwd, bwd)
    serial_cost = sum(prof[(tuple(g), ())] for g in fwd) + sum(prof[((), tuple(g))] for g in bwd)
    plan_path = os.path.join(args.out_dir, "best_result.json")
    dump_plan(blocks, plan_path, alias=alias, bwd_order=[x for g in bwd for x in g])
    if alias:
        print("deferred weight gradients:", sorted(alias.values()), flush=True)
    print(f"predicted: paired {cost:.3f} ms vs unpaired groups {serial_cost:.3f} ms per micro-batch", flush=True)
    print(json.dumps(json.load(open(plan_path))["DCBlocks"]), flush=True)
    ser, dbl = validate(cfg, w, mbs, plan_path)
    print(f"sequence time {ser:.3f} ms  schedule time {dbl:.3f} ms  speedup {ser / dbl:.4f}", flush=True)
    ser0, dbl0 = validate(cfg, w, mbs, None)
    print(f"built-in plan: sequence time {ser0:.3f} ms  schedule time {dbl0:.3f} ms  speedup {ser0 / dbl0:.4f}", flush=True)


if __name__ == "__main__":
    main()
