"""Host logic of the double-strand runtime (no GPU): op vocabulary, plan schema, graph wiring."""
import json

import pytest

from dhellam_amd.core import dstb


def test_op_ids_are_the_reference_vocabulary():
    # dhellam/core/dstb.py:24-58
    expect = dict(ln_attn=1, ln_mlp=2, gemm_attn_column=3, gemm_attn_linear=4, gemm_mlp_column=5, gemm_mlp_linear=6,
                  attn=7, bda_mlp=8, bda_attn=9, reduce_scatter=10, all_gather=11, swiglu=12, gemm_dgrad_mlp_c=13,
                  gemm_wgrad_mlp_c=14, gemm_dgrad_mlp_l=15, gemm_wgrad_mlp_l=16, gemm_dgrad_attn_c=17,
                  gemm_wgrad_attn_c=18, gemm_dgrad_attn_l=19, gemm_wgrad_attn_l=20, gemm_wgrad_mlp_c_n=114,
                  gemm_wgrad_mlp_l_n=116, gemm_wgrad_attn_c_n=118, gemm_wgrad_attn_l_n=120, swiglu_bwd=21,
                  bda_mlp_bwd=22, bda_bwd_attn=23, attn_bwd=24, ln_bwd_mlp=25, ln_bwd_attn=26, ring_attn_fwd=29,
                  ring_attn_bwd=30)
    for k, v in expect.items():
        assert dstb.FuncChoice[k].value == v


def test_default_plans_and_graph_wiring():
    plan = dstb.init_DCBlocks()
    dc, fwd, bwd = plan
    assert len(dc) == 17 and len(fwd) == 11 and len(bwd) == 12          # dstb.py:1043-1060, 1080-1093, 1115-1129
    names = lambda col: [str(o) for o in (col or [])]
    assert names(dc[2].stream1_op) == ["gemm_attn_c", "rope", "fl_attn"] and names(dc[2].stream3_op) == ["allgather_mlp_bwd"]
    assert names(dc[12].stream2_op) == ["gemm_dgrad_attn_l", "gemm_wgrad_attn_l", "attn_bwd", "rope_bwd"]
    ops = plan.ops
    assert [str(o) for o in ops["allgather_mlp_bwd"].get_next_op()] == ["gemm_dgrad_mlp_l", "gemm_wgrad_mlp_l"]
    assert ops["bda_mlp"].get_next_op() == [] and ops["ln_attn_bwd"].get_next_op() == []
    assert ops["allgather_attn"].is_comm == 1 and ops["reduce_scatter_attn_c_bwd"].is_comm == 2
    # every forward op is reachable from ln_attn in chain order
    chain, node = [], ops["ln_attn"]
    while node is not None:
        chain.append(str(node))
        nxt = node.get_next_op()
        node = nxt[0] if nxt else None
    assert chain == ["ln_attn", "allgather_attn", "gemm_attn_c", "rope", "fl_attn", "gemm_attn_l", "reduce_scatter_attn",
                     "bda_attn", "ln_mlp", "allgather_mlp", "gemm_mlp_c", "swiglu_mlp", "gemm_mlp_l",
                     "reduce_scatter_mlp", "bda_mlp"]


def test_plan_file_schema(tmp_path):
    p = {"DCBlocks": [[["ln_attn"], "None", "None"], ["None", "bda_mlp_bwd", ["allgather_attn"]],
                      [["gemm_attn_c", "rope", "fl_attn"], ["gemm_wgrad_mlp_c_n"], "None"]]}
    f = tmp_path / "plan.json"
    f.write_text(json.dumps(p))
    plan = dstb.init_DCBlocks(str(f))
    assert len(plan.dcblocks) == 3 and len(plan.fwd_only) == 11         # missing sections fall back to the built-ins
    assert [str(o) for o in plan.dcblocks[1].stream2_op] == ["bda_mlp_bwd"]
    assert plan.dcblocks[0].stream2_op is None
    assert [str(o) for o in plan.dcblocks[2].stream1_op] == ["gemm_attn_c", "rope", "fl_attn"]   # no second rope inserted
    assert plan.movable == {"gemm_wgrad_mlp_c_n"}
    with pytest.raises(KeyError):
        dstb.init_DCBlocks({"DCBlocks": [[["no_such_op"], "None", "None"]]})
    with pytest.raises(KeyError):
        dstb.init_DCBlocks({"fwd_only": []})
    with pytest.raises(ValueError):
        dstb.init_DCBlocks({"DCBlocks": [[["ln_attn"], "None"]]})


def test_layer_config_derived_sizes():
    from dhellam_amd.core.layer import llama70b_tp8_shard, small_fp32_layer
    c = llama70b_tp8_shard()
    assert (c.head_dim, c.heads_per_rank, c.groups_per_rank, c.ffn_per_rank, c.qkv_per_rank, c.sp_rows, c.tokens) == \
        (128, 8, 1, 3584, 1280, 512, 4096)
    s = small_fp32_layer()
    assert (s.head_dim, s.heads_per_rank, s.groups_per_rank, s.ffn_per_rank, s.qkv_per_rank, s.sp_rows) == \
        (64, 16, 16, 2816, 3072, 1024)


def test_cu_mask_words():
    """Mask words for streams bound to a set of compute units: bit i of word i // 32."""
    from dhellam_amd.common.streams import cu_mask_words
    assert cu_mask_words(256, 0, 248) == [0xFFFFFFFF] * 7 + [0x00FFFFFF]
    assert cu_mask_words(256, 248, 8) == [0] * 7 + [0xFF000000]
    assert cu_mask_words(40, 30, 4) == [0xC0000000, 0x3]
    a, b = cu_mask_words(256, 0, 248), cu_mask_words(256, 248, 8)
    assert all(x & y == 0 and x | y == 0xFFFFFFFF for x, y in zip(a, b))     # a partition of the device
    for bad in ((256, 250, 8), (256, -1, 4), (256, 0, 0)):
        try:
            cu_mask_words(*bad)
        except ValueError:
            continue
        raise AssertionError(bad)
