"""Dynamic programme over op pairings and the plan writer.

Counterpart of search/search.py: ``parse_op_file`` (:61-75), ``dp`` (:77-143) and the JSON
dump (:180-244).  The reference enumerates every refinement of the boundary groups into
exactly m and n groups and runs a 2-D DP for each pair of refinements; the same optimum is
reached here by ONE DP over (forward ops consumed, backward ops consumed) whose moves are
"take the next contiguous forward group", "take the next backward group" or "pair the two",
a group never crossing a boundary.  Profile strings are parsed with ``ast.literal_eval``.
Beyond the reference: ``search_plan_with_parking`` also decides which weight gradients to defer
to a later block under their ``*_n`` placeholders (the runtime and the plan format support
that, dhellam/core/dstb.py:543-598,931-939; the reference's search never proposes it), and the
writer emits the ``fwd_only`` / ``bwd_only`` sections the loader reads.
"""
from __future__ import annotations

import ast
import json
import re
from typing import Dict, List, Sequence, Tuple

from .op_table import COMM_CONSUMER, ID_TO_NAME, PLACEHOLDER_OF, PLAN_NAME

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


def search_plans(profile: Dict[Key, float], fwd_groups: List[List[int]], bwd_groups: List[List[int]],
                 illegal=None, alias=None, k: int = 1) -> List[Tuple[float, List[Tuple[List[int], List[int]]]]]:
    """The ``k`` cheapest sequences of blocks [(fwd group, bwd group)], either possibly empty, that cover both op
    lists in order, by the sum of the blocks' measured times, cheapest first (the reference keeps every plan it
    enumerates as a candidate file for its execute stage, search/execute.py:33-36; here the DP itself carries the k
    best partial plans per cell).  ``illegal(f, b)`` forbids pairing two groups (the reference forbids pairs where
    both sides communicate, search.py:13-21).  ``alias``: {op id: op id whose records time it} (a parked weight
    gradient runs the kernel of the op it was parked from).  Raises KeyError if the profile lacks a needed
    record."""
    F, fs = _starts(fwd_groups)
    B, bs = _starts(bwd_groups)
    nf, nb = len(F), len(B)
    k = max(1, int(k))
    # cell -> up to k entries (cost, (fg, bg), rank of the predecessor entry), cheapest first
    cells = [[[] for _ in range(nb + 1)] for _ in range(nf + 1)]
    cells[0][0] = [(0.0, None, -1)]
    al = alias or {}
    t = lambda f, b: profile[(tuple(al.get(x, x) for x in f), tuple(al.get(x, x) for x in b))]
    for i in range(nf + 1):
        for j in range(nb + 1):
            if i == 0 and j == 0:
                continue
            cand = []
            fgs = [F[a:i] for a in range(fs[i - 1], i)] if i > 0 else []
            bgs = [B[a:j] for a in range(bs[j - 1], j)] if j > 0 else []
            moves = [(fg, []) for fg in fgs] + [([], bg) for bg in bgs]
            moves += [(fg, bg) for fg in fgs for bg in bgs if illegal is None or not illegal(fg, bg)]
            for fg, bg in moves:
                prev = cells[i - len(fg)][j - len(bg)]
                if not prev:
                    continue
                step = t(fg, bg)
                cand.extend((c + step, (fg, bg), r) for r, (c, _, _) in enumerate(prev))
            cand.sort(key=lambda e: e[0])
            cells[i][j] = cand[:k]
    out = []
    for rank in range(len(cells[nf][nb])):
        blocks, i, j, r = [], nf, nb, rank
        total = cells[nf][nb][rank][0]
        while i > 0 or j > 0:
            _, (fg, bg), pr = cells[i][j][r]
            blocks.append((list(fg), list(bg)))
            i, j, r = i - len(fg), j - len(bg), pr
        blocks.reverse()
        out.append((total, blocks))
    return out


def search_plan(profile: Dict[Key, float], fwd_groups: List[List[int]], bwd_groups: List[List[int]],
                illegal=None, alias=None) -> Tuple[float, List[Tuple[List[int], List[int]]]]:
    """The cheapest plan of ``search_plans``: (cost, blocks)."""
    found = search_plans(profile, fwd_groups, bwd_groups, illegal, alias, 1)
    if not found:
        raise KeyError("no plan covers the op lists")
    return found[0]


def park_choices(bwd_groups: List[List[int]], movable: Sequence[int]):
    """Every way of deferring weight gradients: each movable op either stays, or leaves its place and runs as a
    group of its own right after a LATER boundary group (where its ``*_n`` placeholder then sits,
    dhellam/core/dstb.py:543-598).  Yields (modified backward groups, {placeholder id: op id}); the group an op
    leaves is cut in two at its place."""
    where = {op: gi for gi, g in enumerate(bwd_groups) for op in g}
    movable = [m for m in movable if m in where]
    options = [[None] + list(range(where[m] + 1, len(bwd_groups))) for m in movable]

    def rec(k, chosen):
        if k == len(movable):
            yield dict(chosen)
            return
        for o in options[k]:
            chosen.append((movable[k], o))
            yield from rec(k + 1, chosen)
            chosen.pop()

    for choice in rec(0, []):
        groups, alias = [], {}
        after = {}
        for m, o in choice.items():
            if o is not None:
                after.setdefault(o, []).append(m)
        for gi, g in enumerate(bwd_groups):
            cur = []
            for op in g:
                if choice.get(op) is not None:
                    if cur:
                        groups.append(cur)
                    cur = []
                else:
                    cur.append(op)
            if cur:
                groups.append(cur)
            for m in after.get(gi, []):
                groups.append([PLACEHOLDER_OF[m]])
                alias[PLACEHOLDER_OF[m]] = m
        yield groups, alias


def search_candidates_with_parking(profile: Dict[Key, float], fwd_groups, bwd_groups, movable=None, illegal=None,
                                   k: int = 1):
    """``search_plans`` over every choice of deferred weight gradients: the ``k`` cheapest (cost, blocks, alias)
    overall, cheapest first.  In the blocks a deferred op appears as its placeholder id at the place where it
    runs; ``alias`` maps the placeholders used to the ops they defer (``plan_to_json`` puts the op's own name back
    where it was parked)."""
    movable = list(PLACEHOLDER_OF) if movable is None else list(movable)
    found = []
    for groups, alias in park_choices(bwd_groups, movable):
        try:
            for cost, blocks in search_plans(profile, fwd_groups, groups, illegal, alias, k):
                found.append((cost, blocks, alias))
        except KeyError:
            continue                      # the profile has no record for a group this choice needs
    if not found:
        raise KeyError("the profile lacks the records of every candidate plan")
    found.sort(key=lambda e: e[0])
    return found[:max(1, int(k))]


def search_plan_with_parking(profile: Dict[Key, float], fwd_groups, bwd_groups, movable=None, illegal=None):
    """The cheapest of ``search_candidates_with_parking``: (cost, blocks, alias)."""
    return search_candidates_with_parking(profile, fwd_groups, bwd_groups, movable, illegal, 1)[0]


def plan_to_json(blocks, with_comm_standins: bool = True, alias=None, bwd_order: Sequence[int] = ()) -> dict:
    """{"DCBlocks": [...], "fwd_only": [...], "bwd_only": [...]}, each a list of
    [stream1, stream2, stream3] in the reference's schema (writer search.py:180-244, reader
    dhellam/core/dstb.py:901-1041): op-name lists, or the string "None" for an empty column.  The
    sequence-parallel stand-in ops go into the third column of the block that holds their
    consumer.  ``fwd_only`` / ``bwd_only`` (the schedules of the first forward and the last
    backward) hold the same groups in the same order, one strand each.
    ``alias`` ({placeholder id: deferred op id}, from ``search_plan_with_parking``) with ``bwd_order`` (the
    backward ops in their original order): a deferred op is named again right after the op it followed, where
    the runtime parks it, and its placeholder stays where the search put it."""
    comm_of = {}
    for comm, consumer in COMM_CONSUMER.items():
        comm_of.setdefault(consumer, []).append(comm)
    nm = lambda i: PLAN_NAME.get(ID_TO_NAME[i], ID_TO_NAME[i])
    blocks = [(list(f), list(b)) for f, b in blocks]
    for ph, op in (alias or {}).items():
        order = list(bwd_order)
        k = order.index(op)
        placed = False
        for prev in reversed(order[:k]):                  # nearest earlier op that is still at its place
            for _, bg in blocks:
                if prev in bg:
                    bg.insert(bg.index(prev) + 1, op)
                    placed = True
                    break
            if placed:
                break
        if not placed:                                    # nothing before it: park it in the first backward block
            next(bg for _, bg in blocks if bg).insert(0, op)

    def section(blks):
        out = []
        for fg, bg in blks:
            first, second = [nm(i) for i in fg], [nm(i) for i in bg]
            third = [c for op in first + second for c in comm_of.get(op, [])] if with_comm_standins else []
            out.append([first or "None", second or "None", third or "None"])
        return out

    return {"DCBlocks": section(blocks),
            "fwd_only": section([(f, []) for f, _ in blocks if f]),
            "bwd_only": section([([], b) for _, b in blocks if b])}


def unpaired_cost(profile: Dict[Key, float], fwd_groups, bwd_groups) -> Tuple[float, float]:
    """(forward alone, backward alone): the boundary groups one after the other on their own, which is what the
    ``fwd_only`` and ``bwd_only`` sections of a plan run for the first forward and the last backward."""
    return (sum(profile[(tuple(g), ())] for g in fwd_groups), sum(profile[((), tuple(g))] for g in bwd_groups))


def dump_plan(blocks, path: str, alias=None, bwd_order: Sequence[int] = ()) -> dict:
    data = plan_to_json(blocks, alias=alias, bwd_order=bwd_order)
    with open(path, "w") as f:
        json.dump(data, f, indent=4)
    return data
