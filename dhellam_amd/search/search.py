"""Dynamic programme over op pairings and the plan writer.

Counterpart of search/search.py: ``parse_op_file`` (:61-75), ``dp`` (:77-143) and the JSON
dump (:180-244).  The reference enumerates every refinement of the boundary groups into
exactly m and n groups and runs a 2-D DP for each pair of refinements; the same optimum is
reached here by ONE DP over (forward ops consumed, backward ops consumed) whose moves are
"take the next contiguous forward group", "take the next backward group" or "pair the two",
a group never crossing a boundary.  Profile strings are parsed with ``ast.literal_eval``.
"""
from __future__ import annotations

import ast
import json
import re
from typing import Dict, List, Sequence, Tuple

from .op_table import COMM_CONSUMER, ID_TO_NAME, PLAN_NAME

Key = Tuple[Tuple[int, ...], Tuple[int, ...]]
_LINE = re.compile(r'\[\s*(\[[\d,\s]*\])\s*,\s*(\[[\d,\s]*\])\s*\]\s*speedup:\s*([0-9.eE+-]+)\s*'
                   r'seq_time:\s*([0-9.eE+-]+)\s*para_time:\s*([0-9.eE+-]+)')


def format_record(fwd_ids: Sequence[int], bwd_ids: Sequence[int], speedup: float, seq_time: float, para_time: float) -> str:
    """One line of op_profile_num.txt (search/profiler.py:179-180)."""
    return f"[{list(fwd_ids)},{list(bwd_ids)}] speedup: {speedup} seq_time:{seq_time} para_time:{para_time}\n"


def parse_op_file(path: str) -> Dict[Key, float]:
    """{(fwd ids, bwd ids): para_time in ms}; a later line for the same pair wins."""
    out: Dict[Key, float] = {}
    with open(path) as f:
        for line in f:
            m = _LINE.match(line.strip())
            if not m:
                if line.strip():
                    print(f"line:{line.rstrip()} is not match")
                continue
            out[(tuple(ast.literal_eval(m.group(1))), tuple(ast.literal_eval(m.group(2))))] = float(m.group(5))
    return out


def _starts(groups: List[List[int]]):
    """For a position i in the flattened op list: the position where its boundary group starts."""
    flat, start = [], []
    for g in groups:
        s = len(flat)
        for op in g:
            flat.append(op)
            start.append(s)
    return flat, start


def search_plan(profile: Dict[Key, float], fwd_groups: List[List[int]], bwd_groups: List[List[int]],
                illegal=None) -> Tuple[float, List[Tuple[List[int], List[int]]]]:
    """Best sequence of blocks [(fwd group, bwd group)], either possibly empty, that covers
    both op lists in order and minimises the sum of the blocks' measured times.  ``illegal(f, b)``
    forbids pairing two groups (the reference forbids pairs where both sides communicate,
    search.py:13-21).  Raises KeyError if the profile lacks a needed record."""
    F, fs = _starts(fwd_groups)
    B, bs = _starts(bwd_groups)
    nf, nb = len(F), len(B)
    INF = float("inf")
    cost = [[INF] * (nb + 1) for _ in range(nf + 1)]
    back = [[None] * (nb + 1) for _ in range(nf + 1)]
    cost[0][0] = 0.0
    t = lambda f, b: profile[(tuple(f), tuple(b))]
    for i in range(nf + 1):
        for j in range(nb + 1):
            if i == 0 and j == 0:
                continue
            best, arg = INF, None
            fgs = [F[a:i] for a in range(fs[i - 1], i)] if i > 0 else []
            bgs = [B[a:j] for a in range(bs[j - 1], j)] if j > 0 else []
            for fg in fgs:
                c = cost[i - len(fg)][j] + t(fg, [])
                if c < best:
                    best, arg = c, (fg, [])
            for bg in bgs:
                c = cost[i][j - len(bg)] + t([], bg)
                if c < best:
                    best, arg = c, ([], bg)
            for fg in fgs:
                for bg in bgs:
                    if illegal is not None and illegal(fg, bg):
                        continue
                    c = cost[i - len(fg)][j - len(bg)] + t(fg, bg)
                    if c < best:
                        best, arg = c, (fg, bg)
            cost[i][j], back[i][j] = best, arg
    blocks = []
    i, j = nf, nb
    while i > 0 or j > 0:
        fg, bg = back[i][j]
        blocks.append((list(fg), list(bg)))
        i -= len(fg)
        j -= len(bg)
    blocks.reverse()
    return cost[nf][nb], blocks


def plan_to_json(blocks, with_comm_standins: bool = True) -> dict:
    """{"DCBlocks": [[stream1, stream2, stream3], ...]} in the reference's schema
    (search.py:180-244): op-name lists, or the string "None" for an empty column.  The
    sequence-parallel stand-in ops go into the third column of the block that holds their
    consumer."""
    comm_of = {}
    for comm, consumer in COMM_CONSUMER.items():
        comm_of.setdefault(consumer, []).append(comm)
    out = []
    for fg, bg in blocks:
        names = lambda ids: [PLAN_NAME.get(ID_TO_NAME[i], ID_TO_NAME[i]) for i in ids]
        first, second = names(fg), names(bg)
        third = [c for op in first + second for c in comm_of.get(op, [])] if with_comm_standins else []
        out.append([first or "None", second or "None", third or "None"])
    return {"DCBlocks": out}


def dump_plan(blocks, path: str) -> dict:
    data = plan_to_json(blocks)
    with open(path, "w") as f:
        json.dump(data, f, indent=4)
    return data
