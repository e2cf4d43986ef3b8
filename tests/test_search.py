"""Plan search host logic (no GPU): record format, DP optimality against brute force, plan JSON."""
import itertools
import random

from dhellam_amd.core import dstb
from dhellam_amd.search import op_table, search


def test_op_ids_and_candidates():
    assert op_table.OP_TABLE_IDX["ln_attn"] == 24 and op_table.OP_TABLE_IDX["attn_bwd"] == 10      # search/op_table.py:1-37
    assert op_table.OP_TABLE_IDX["gemm_wgrad_mlp_c_reduce_scatter_mlp_c_bwd"] == 9
    fwd_c, bwd_c = op_table.get_candidate_operator_groups()
    assert fwd_c[0] == [] and [24] in fwd_c and [16, 35, 11, 17] in fwd_c and [35, 11] in fwd_c
    assert [16, 11] not in fwd_c                                   # not contiguous
    assert [24, 16] not in fwd_c                                   # crosses a boundary
    assert len(fwd_c) == 1 + 1 + 10 + 3 + 6 + 1 and len(bwd_c) == 1 + 1 + 10 + 1 + 3 + 15 + 1 + 1


def test_record_format_roundtrip(tmp_path):
    f = tmp_path / "op_profile_num.txt"
    with open(f, "w") as fp:
        fp.write(search.format_record([16, 35, 11], [19, 23], 1.25, 2.5, 2.0))
        fp.write(search.format_record([], [26], 1.0, 0.5, 0.5))
        fp.write(search.format_record([24], [], 1.0, 0.25, 0.25))
        fp.write("garbage line\n")
    assert open(f).readline() == "[[16, 35, 11],[19, 23]] speedup: 1.25 seq_time:2.5 para_time:2.0\n"   # profiler.py:179-180
    prof = search.parse_op_file(str(f))
    assert prof == {((16, 35, 11), (19, 23)): 2.0, ((), (26,)): 0.5, ((24,), ()): 0.25}


def _brute(profile, fwd_groups, bwd_groups):
    """Reference-style search: enumerate every refinement of the boundary groups, then the
    classic 2-D DP over the two group sequences (search/search.py:77-143)."""
    def refinements(groups):
        per = []
        for g in groups:
            opts = []
            for cuts in itertools.product([0, 1], repeat=len(g) - 1):
                parts, cur = [], [g[0]]
                for op, cut in zip(g[1:], cuts):
                    if cut:
                        parts.append(cur); cur = [op]
                    else:
                        cur.append(op)
                parts.append(cur)
                opts.append(parts)
            per.append(opts)
        for combo in itertools.product(*per):
            yield [p for parts in combo for p in parts]
    best = float("inf")
    t = lambda f, b: profile[(tuple(f), tuple(b))]
    for fr in refinements(fwd_groups):
        for br in refinements(bwd_groups):
            m, n = len(fr), len(br)
            d = [[0.0] * (n + 1) for _ in range(m + 1)]
            for i in range(1, m + 1):
                d[i][0] = d[i - 1][0] + t(fr[i - 1], [])
            for j in range(1, n + 1):
                d[0][j] = d[0][j - 1] + t([], br[j - 1])
            for i in range(1, m + 1):
                for j in range(1, n + 1):
                    d[i][j] = min(d[i - 1][j] + t(fr[i - 1], []), d[i][j - 1] + t([], br[j - 1]),
                                  d[i - 1][j - 1] + t(fr[i - 1], br[j - 1]))
            best = min(best, d[m][n])
    return best


def test_dp_matches_brute_force_enumeration():
    rng = random.Random(0)
    fwd_groups, bwd_groups = [[1], [2, 3, 4], [5, 6]], [[11, 12], [13], [14, 15, 16]]
    for trial in range(5):
        prof = {}
        fc, bc = op_table.candidate_groups(fwd_groups), op_table.candidate_groups(bwd_groups)
        solo = {}
        for f in fc:
            for b in bc:
                if not f and not b:
                    continue
                base = sum(solo.setdefault(x, rng.uniform(0.1, 1.0)) for x in f + b)
                # pairing saves a random share of the smaller side
                save = rng.uniform(0, 0.9) * min(sum(solo[x] for x in f), sum(solo[x] for x in b)) if f and b else 0.0
                prof[(tuple(f), tuple(b))] = base - save
        cost, blocks = search.search_plan(prof, fwd_groups, bwd_groups)
        assert abs(cost - _brute(prof, fwd_groups, bwd_groups)) < 1e-9
        # the blocks cover both lists in order and their times add up to the cost
        assert [x for f, _ in blocks for x in f] == [1, 2, 3, 4, 5, 6]
        assert [x for _, b in blocks for x in b] == [11, 12, 13, 14, 15, 16]
        assert abs(sum(prof[(tuple(f), tuple(b))] for f, b in blocks) - cost) < 1e-9


def test_illegal_pairs_are_never_chosen():
    fwd_groups, bwd_groups = [[1, 2]], [[11, 12]]
    prof = {(tuple(f), tuple(b)): 1.0 for f in op_table.candidate_groups(fwd_groups)
            for b in op_table.candidate_groups(bwd_groups) if f or b}
    prof[((1, 2), (11, 12))] = 0.1
    cost, blocks = search.search_plan(prof, fwd_groups, bwd_groups)
    assert blocks == [([1, 2], [11, 12])] and cost == 0.1
    cost, blocks = search.search_plan(prof, fwd_groups, bwd_groups, illegal=lambda f, b: len(f) == 2 and len(b) == 2)
    assert cost == 1.0 + 1.0 - 0.0 or cost == 2.0
    assert ([1, 2], [11, 12]) not in blocks


def test_plan_json_is_loadable_and_complete(tmp_path):
    (_, _, fwd), (_, _, bwd) = op_table.operator_list_prune()
    # a plan that pairs group by group where possible
    blocks = [(fwd[i] if i < len(fwd) else [], bwd[i] if i < len(bwd) else []) for i in range(max(len(fwd), len(bwd)))]
    data = search.dump_plan(blocks, str(tmp_path / "best_result.json"))
    assert set(data) == {"DCBlocks", "fwd_only", "bwd_only"} and all(len(b) == 3 for b in data["DCBlocks"])
    assert data["DCBlocks"][0] == [["ln_attn"], ["bda_mlp_bwd"], "None"]
    assert data["DCBlocks"][1][2] == ["allgather_attn", "allgather_mlp_bwd"]
    assert data["DCBlocks"][2][1] == ["gemm_wgrad_mlp_c"]                      # fused search op written under its plan name
    plan = dstb.init_DCBlocks(str(tmp_path / "best_result.json"))
    named = [str(o) for blk in plan.dcblocks for col in (blk.stream1_op, blk.stream2_op, blk.stream3_op) for o in (col or [])]
    graph_ops = [n for n, num, *_ in dstb._GRAPH if num < 100]
    assert sorted(named) == sorted(graph_ops), "every op of the layer appears exactly once in the plan"
    # a comm stand-in never precedes its producer's block and sits in its consumer's block
    pos = {str(o): i for i, blk in enumerate(plan.dcblocks) for col in (blk.stream1_op, blk.stream2_op, blk.stream3_op) for o in (col or [])}
    for comm, consumer in op_table.COMM_CONSUMER.items():
        assert pos[comm] == pos[consumer] and pos[str(plan.ops[comm].pre)] < pos[comm]


def _ops_of(blocks, col):
    return [str(o) for blk in blocks for o in (getattr(blk, col) or [])]


def test_plan_writer_emits_fwd_only_and_bwd_only_sections(tmp_path):
    """The writer's three sections round-trip through the loader: fwd_only holds every forward op once, in order,
    with nothing in the backward column; bwd_only the mirror image; stand-in collectives ride with their consumers."""
    (_, _, fwd), (_, _, bwd) = op_table.operator_list_prune()
    blocks = [(fwd[i] if i < len(fwd) else [], bwd[i] if i < len(bwd) else []) for i in range(max(len(fwd), len(bwd)))]
    data = search.dump_plan(blocks, str(tmp_path / "p.json"))
    assert all(b[1] == "None" for b in data["fwd_only"]) and all(b[0] == "None" for b in data["bwd_only"])
    assert len(data["fwd_only"]) == len(fwd) and len(data["bwd_only"]) == len(bwd)
    plan = dstb.init_DCBlocks(str(tmp_path / "p.json"))
    name = lambda i: op_table.PLAN_NAME.get(op_table.ID_TO_NAME[i], op_table.ID_TO_NAME[i])
    assert _ops_of(plan.fwd_only, "stream1_op") == [name(i) for g in fwd for i in g]
    assert _ops_of(plan.bwd_only, "stream2_op") == [name(i) for g in bwd for i in g]
    assert sorted(_ops_of(plan.fwd_only, "stream3_op")) == sorted(c for c in op_table.COMM_CONSUMER if not c.endswith("_bwd"))
    assert sorted(_ops_of(plan.bwd_only, "stream3_op")) == sorted(c for c in op_table.COMM_CONSUMER if c.endswith("_bwd"))


def _synthetic_profile(fwd_groups, bwd_groups, rng, cheap_pair=None):
    solo, prof = {}, {}
    for f in op_table.candidate_groups(fwd_groups):
        for b in op_table.candidate_groups(bwd_groups):
            if not f and not b:
                continue
            base = sum(solo.setdefault(x, rng.uniform(0.1, 1.0)) for x in f + b)
            save = rng.uniform(0, 0.9) * min(sum(solo[x] for x in f), sum(solo[x] for x in b)) if f and b else 0.0
            prof[(tuple(f), tuple(b))] = base - save
    return prof, solo


def test_parking_search_matches_brute_force_over_every_choice():
    """The deferred-weight-gradient search against the reference-style enumeration run on every park choice."""
    rng = random.Random(1)
    W1, W2 = 12, 15
    fwd_groups, bwd_groups = [[1], [2, 3], [4]], [[11, W1, 13], [14], [W2], [16]]
    saved = dict(op_table.PLACEHOLDER_OF)
    op_table.PLACEHOLDER_OF.clear()
    op_table.PLACEHOLDER_OF.update({W1: 912, W2: 915})
    search.PLACEHOLDER_OF = op_table.PLACEHOLDER_OF
    try:
        for trial in range(4):
            prof, _ = _synthetic_profile(fwd_groups, bwd_groups, rng)
            cost, blocks, alias = search.search_plan_with_parking(prof, fwd_groups, bwd_groups)
            best = float("inf")
            n_choices = 0
            for groups, al in search.park_choices(bwd_groups, [W1, W2]):
                n_choices += 1
                p2 = dict(prof)
                for (f, b), v in prof.items():            # the placeholder runs the kernel of the op it defers
                    for ph, op in al.items():
                        if b == (op,):
                            p2[(f, (ph,))] = v
                best = min(best, _brute(p2, fwd_groups, groups))
            assert n_choices == 4 * 2                     # W1: stay or after group 1, 2, 3; W2: stay or after group 3
            assert abs(cost - best) < 1e-9
            no_parking, _ = search.search_plan(prof, fwd_groups, bwd_groups)
            assert cost <= no_parking + 1e-12
            ran = [alias.get(x, x) for _, b in blocks for x in b]
            assert sorted(ran) == [11, 12, 13, 14, 15, 16]
    finally:
        op_table.PLACEHOLDER_OF.clear()
        op_table.PLACEHOLDER_OF.update(saved)


def test_parked_plan_names_the_op_where_it_is_parked_and_its_placeholder_where_it_runs(tmp_path):
    (_, _, fwd), (_, _, bwd) = op_table.operator_list_prune()
    n = op_table.OP_TABLE_IDX
    w = n["gemm_wgrad_mlp_l"]
    # hand-made result of the search: the mlp_l weight gradient leaves its group and runs after the 4th group
    groups, alias = next((g, a) for g, a in search.park_choices(bwd, [w]) if a and g.index([n["gemm_wgrad_mlp_l_n"]]) == 5)
    blocks = [(fwd[i] if i < len(fwd) else [], groups[i] if i < len(groups) else []) for i in range(max(len(fwd), len(groups)))]
    order = [x for g in bwd for x in g]
    data = search.dump_plan(blocks, str(tmp_path / "p.json"), alias=alias, bwd_order=order)
    col2 = [b[1] for b in data["DCBlocks"]]
    assert col2[1] == ["gemm_dgrad_mlp_l", "gemm_wgrad_mlp_l"]          # parked right after the op it followed
    assert ["gemm_wgrad_mlp_l_n"] in col2
    plan = dstb.init_DCBlocks(str(tmp_path / "p.json"))
    assert plan.movable == {"gemm_wgrad_mlp_l_n"}
    flat = _ops_of(plan.dcblocks, "stream2_op")
    assert flat.index("gemm_wgrad_mlp_l") < flat.index("gemm_wgrad_mlp_l_n")
    assert "gemm_wgrad_mlp_l_n" in _ops_of(plan.bwd_only, "stream2_op")


def test_context_parallel_groups_and_graph():
    """cp = 4: ring steps replace fl_attn / attn_bwd in the boundary groups, the graph and the built-in plans."""
    (nf, _, fwd), (nb, _, bwd) = op_table.operator_list_prune(4)
    n = op_table.OP_TABLE_IDX
    assert n["cp_attn_block_fwd_1"] == 30 and n["cp_attn_block_bwd_3"] == 34                      # search/op_table.py:31-36
    assert [n["cp_attn_block_fwd_1"]] in fwd and [n["cp_attn_block_fwd_4"], n["gemm_attn_l"]] in fwd
    assert [n["cp_attn_block_bwd_5"], n["gemm_dgrad_attn_c"]] in bwd and [n["cp_attn_block_bwd_4"]] in bwd
    assert all(n["fl_attn"] not in g and n["rope"] not in g for g in fwd)
    (_, _, f2), (_, _, b2) = op_table.operator_list_prune(2)
    assert [30] in f2 and [31, 17] in f2 and [32] in b2 and [33] in b2 and [34, 6] in b2           # op_table.py:68-89
    plan = dstb.init_DCBlocks(None, context_parallel_size=4)
    fl = _ops_of(plan.fwd_only, "stream1_op")
    assert fl[fl.index("gemm_attn_c") + 1: fl.index("gemm_attn_l")] == [f"cp_attn_block_fwd_{i}" for i in range(1, 5)]
    bl = _ops_of(plan.bwd_only, "stream2_op")
    i0 = bl.index("cp_attn_block_bwd_1")
    assert bl[i0:i0 + 5] == [f"cp_attn_block_bwd_{i}" for i in range(1, 6)] and "attn_bwd" not in bl and "rope_bwd" not in bl
    assert plan.ops["gemm_attn_l"].pre is plan.ops["cp_attn_block_fwd_4"]
    assert plan.ops["gemm_wgrad_attn_c"].pre is plan.ops["cp_attn_block_bwd_5"]
    # a searched plan over these groups loads
    blocks = [(fwd[i] if i < len(fwd) else [], bwd[i] if i < len(bwd) else []) for i in range(max(len(fwd), len(bwd)))]
    loaded = dstb.init_DCBlocks(search.plan_to_json(blocks), context_parallel_size=4)
    assert "cp_attn_block_bwd_5" in _ops_of(loaded.dcblocks, "stream2_op")


def _all_plan_costs(profile, fwd_groups, bwd_groups):
    """Cost of EVERY plan (every block sequence that covers both lists in order with groups inside the
    boundaries), by plain recursion: the ground truth for the k-best DP."""
    F, fs = search._starts(fwd_groups)
    B, bs = search._starts(bwd_groups)
    t = lambda f, b: profile[(tuple(f), tuple(b))]
    out = []

    def rec(i, j, acc):
        if i == 0 and j == 0:
            out.append(acc)
            return
        fgs = [F[a:i] for a in range(fs[i - 1], i)] if i > 0 else []
        bgs = [B[a:j] for a in range(bs[j - 1], j)] if j > 0 else []
        for fg in fgs:
            rec(i - len(fg), j, acc + t(fg, []))
        for bg in bgs:
            rec(i, j - len(bg), acc + t([], bg))
        for fg in fgs:
            for bg in bgs:
                rec(i - len(fg), j - len(bg), acc + t(fg, bg))

    rec(len(F), len(B), 0.0)
    return sorted(out)


def test_k_best_plans_are_the_k_cheapest_of_all():
    rng = random.Random(1)
    fwd_groups, bwd_groups = [[1], [2, 3]], [[11, 12], [13]]
    fc, bc = op_table.candidate_groups(fwd_groups), op_table.candidate_groups(bwd_groups)
    prof = {(tuple(f), tuple(b)): rng.uniform(0.1, 1.0) for f in fc for b in bc if f or b}
    truth = _all_plan_costs(prof, fwd_groups, bwd_groups)
    for k in (1, 3, 7, len(truth) + 5):
        found = search.search_plans(prof, fwd_groups, bwd_groups, k=k)
        assert len(found) == min(k, len(truth))
        assert all(abs(c - w) < 1e-12 for (c, _), w in zip(found, truth))
        seen = set()
        for cost, blocks in found:
            assert [x for f, _ in blocks for x in f] == [1, 2, 3] and [x for _, b in blocks for x in b] == [11, 12, 13]
            assert abs(sum(prof[(tuple(f), tuple(b))] for f, b in blocks) - cost) < 1e-12
            seen.add(str(blocks))
        assert len(seen) == len(found), "the k plans are k different plans"


def test_execute_stage_keeps_the_measured_winner(tmp_path, monkeypatch):
    """search/execute.py:54-116: every candidate is replayed, the fastest is copied to best.json; the built-in plan
    is always among the candidates and wins ties, so the emitted plan is never slower than running without one."""
    import json
    from dhellam_amd.search import execute as ex
    times = {"a": (10.0, 9.0), "b": (8.5, 9.5), ex.BUILTIN: (9.2, 9.3)}          # (free-running, lockstep)

    def fake_replay(cfg, weights, mbs, plan, steps=20, warmup=3, lockstep=False):
        name = ex.BUILTIN if plan is None else plan["name"]
        return times[name][1 if lockstep else 0]

    monkeypatch.setattr(ex, "replay", fake_replay)
    monkeypatch.setattr(ex, "replay_serial", lambda *a, **k: 9.4)
    cands = [{"name": n, "plan": {"name": n, "DCBlocks": []}, "paired_ms": 2.0} for n in ("a", "b")]
    rep = ex.execute(None, None, [0, 1, 2, 3], cands, str(tmp_path), fwd_alone_ms=1.0, bwd_alone_ms=2.0, log=lambda m: None)
    assert [r["name"] for r in rep["candidates"]] == ["a", "b", ex.BUILTIN]        # the built-in plan was added
    assert rep["best"] == {"name": "b", "lockstep_blocks": False, "ms": 8.5}
    assert rep["candidates"][0]["predicted_lockstep_ms"] == 1.0 + 3 * 2.0 + 2.0
    assert json.load(open(tmp_path / "best.json"))["name"] == "b"
    assert json.load(open(tmp_path / "execute_report.json"))["speedup_over_serial"] == round(9.4 / 8.5, 4)
    # a candidate that only ties with the built-in plan does not displace it, and the built-in plan is written out
    times["a"], times["b"] = (10.0, 9.6), (9.2, 9.5)
    rep = ex.execute(None, None, [0, 1], cands, str(tmp_path), log=lambda m: None)
    assert rep["best"]["name"] == ex.BUILTIN
    written = json.load(open(tmp_path / "best.json"))
    assert written == ex.builtin_plan() and dstb.init_DCBlocks(written).dcblocks
    # lockstep wins where it is the faster mode
    times["a"] = (10.0, 8.0)
    rep = ex.execute(None, None, [0, 1], cands, None, log=lambda m: None)
    assert rep["best"] == {"name": "a", "lockstep_blocks": True, "ms": 8.0}
