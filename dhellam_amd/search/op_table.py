"""Op vocabulary of the plan search and the pre-pruned group boundaries.

Counterpart of search/op_table.py: ``OP_TABLE_IDX`` (:1-37, the ids stored in
``op_profile_num.txt``), ``operator_list_prune`` (:42-92) and
``get_candidate_operator_groups`` (:405-420).  On one GPU there is no communication to
hide, so the communication ops are not search variables: the boundary groups are the
reference's compute groups, with the two RoPE ops added next to the attention ops (or, with
context parallelism, the ring steps in their place), and the
sequence-parallel stand-in ops are attached to the block of their consumer when a plan is
written (search.plan_to_json).
"""
from __future__ import annotations

OP_TABLE_IDX = {
    'allgather_attn': 0, 'allgather_attn_bwd': 1, 'allgather_mlp': 2, 'allgather_mlp_bwd': 3,
    'reduce_scatter_attn': 4, 'reduce_scatter_mlp': 5, 'gemm_dgrad_attn_c': 6, 'gemm_dgrad_mlp_c': 7,
    'gemm_wgrad_attn_c_reduce_scatter_attn_c_bwd': 8, 'gemm_wgrad_mlp_c_reduce_scatter_mlp_c_bwd': 9,
    'attn_bwd': 10, 'fl_attn': 11, 'bda_attn': 12, 'bda_mlp': 13, 'bda_attn_bwd': 14, 'bda_mlp_bwd': 15,
    'gemm_attn_c': 16, 'gemm_attn_l': 17, 'gemm_dgrad_attn_l': 18, 'gemm_dgrad_mlp_l': 19, 'gemm_mlp_c': 20,
    'gemm_mlp_l': 21, 'gemm_wgrad_attn_l': 22, 'gemm_wgrad_mlp_l': 23, 'ln_attn': 24, 'ln_mlp': 25,
    'ln_attn_bwd': 26, 'ln_mlp_bwd': 27, 'swiglu_bwd': 28, 'swiglu_mlp': 29,
    'cp_attn_block_fwd_1': 30, 'cp_attn_block_fwd_2': 31, 'cp_attn_block_bwd_1': 32, 'cp_attn_block_bwd_2': 33,
    'cp_attn_block_bwd_3': 34,
    'rope': 35, 'rope_bwd': 36,                  # not in the reference
}
# Ring steps beyond the five names the reference's table holds (it is written for cp = 2): forward step k >= 3
# gets id 100 + k, backward call k >= 4 gets id 200 + k.
for _k in range(3, 17):
    OP_TABLE_IDX[f'cp_attn_block_fwd_{_k}'] = 100 + _k
for _k in range(4, 18):
    OP_TABLE_IDX[f'cp_attn_block_bwd_{_k}'] = 200 + _k
# Deferred weight-gradient placeholders (dhellam/core/dstb.py:45-48,551-598; plan names string_to_OP :886-889).
# The reference's search never proposes them; here they are search variables (search.search_plan_with_parking),
# with ids of their own.
for _k, _n in enumerate(('gemm_wgrad_mlp_c_n', 'gemm_wgrad_mlp_l_n', 'gemm_wgrad_attn_c_n', 'gemm_wgrad_attn_l_n')):
    OP_TABLE_IDX[_n] = 40 + _k
ID_TO_NAME = {v: k for k, v in OP_TABLE_IDX.items()}
# search id of a weight-gradient op -> search id of its placeholder
PLACEHOLDER_OF = {OP_TABLE_IDX['gemm_wgrad_mlp_c_reduce_scatter_mlp_c_bwd']: OP_TABLE_IDX['gemm_wgrad_mlp_c_n'],
                  OP_TABLE_IDX['gemm_wgrad_mlp_l']: OP_TABLE_IDX['gemm_wgrad_mlp_l_n'],
                  OP_TABLE_IDX['gemm_wgrad_attn_c_reduce_scatter_attn_c_bwd']: OP_TABLE_IDX['gemm_wgrad_attn_c_n'],
                  OP_TABLE_IDX['gemm_wgrad_attn_l']: OP_TABLE_IDX['gemm_wgrad_attn_l_n']}

# Plan-file name of a search op: the reference fuses the column wgrads with the reduce-scatter
# that follows them into one search op and splits the name again when it writes the plan
# (search/search.py:189-193).
PLAN_NAME = {'gemm_wgrad_attn_c_reduce_scatter_attn_c_bwd': 'gemm_wgrad_attn_c',
             'gemm_wgrad_mlp_c_reduce_scatter_mlp_c_bwd': 'gemm_wgrad_mlp_c'}

# stand-in comm op -> the compute op that consumes its result
COMM_CONSUMER = {'allgather_attn': 'gemm_attn_c', 'reduce_scatter_attn': 'bda_attn', 'allgather_mlp': 'gemm_mlp_c',
                 'reduce_scatter_mlp': 'bda_mlp', 'allgather_mlp_bwd': 'gemm_dgrad_mlp_l',
                 'reduce_scatter_mlp_c_bwd': 'ln_mlp_bwd', 'allgather_attn_bwd': 'gemm_dgrad_attn_l',
                 'reduce_scatter_attn_c_bwd': 'ln_attn_bwd'}


def operator_list_prune(context_parallel_size: int = 1):
    """Boundary groups (lists of op ids).  Returns ((min groups, max groups, fwd list),
    (min groups, max groups, bwd list)) like the reference."""
    cp = int(context_parallel_size)
    if not 1 <= cp <= 16:
        raise ValueError(f"context_parallel_size={cp} outside [1, 16]")
    n = OP_TABLE_IDX
    if cp == 1:
        attn_fwd = [[n['gemm_attn_c'], n['rope'], n['fl_attn'], n['gemm_attn_l']]]
        attn_bwd = [[n['gemm_dgrad_attn_l'], n['gemm_wgrad_attn_l'], n['attn_bwd'], n['rope_bwd'], n['gemm_dgrad_attn_c']]]
    else:
        # every ring step but the last posts an exchange in the reference, which makes it a group of its own
        # (op_table.py:68-89 for cp = 2); the last step joins the GEMM that follows it
        f = [n[f'cp_attn_block_fwd_{i}'] for i in range(1, cp + 1)]
        b = [n[f'cp_attn_block_bwd_{i}'] for i in range(1, cp + 2)]
        attn_fwd = [[n['gemm_attn_c']]] + [[i] for i in f[:-1]] + [[f[-1], n['gemm_attn_l']]]
        attn_bwd = [[n['gemm_dgrad_attn_l'], n['gemm_wgrad_attn_l']]] + [[i] for i in b[:-1]] + [[b[-1], n['gemm_dgrad_attn_c']]]
    fwd = [[n['ln_attn']],
           *attn_fwd,
           [n['bda_attn'], n['ln_mlp']],
           [n['gemm_mlp_c'], n['swiglu_mlp'], n['gemm_mlp_l']],
           [n['bda_mlp']]]
    bwd = [[n['bda_mlp_bwd']],
           [n['gemm_dgrad_mlp_l'], n['gemm_wgrad_mlp_l'], n['swiglu_bwd'], n['gemm_dgrad_mlp_c']],
           [n['gemm_wgrad_mlp_c_reduce_scatter_mlp_c_bwd']],
           [n['ln_mlp_bwd'], n['bda_attn_bwd']],
           *attn_bwd,
           [n['gemm_wgrad_attn_c_reduce_scatter_attn_c_bwd']],
           [n['ln_attn_bwd']]]
    cnt = lambda l: sum(len(g) for g in l)
    return (len(fwd), cnt(fwd), fwd), (len(bwd), cnt(bwd), bwd)


def candidate_groups(groups):
    """Every contiguous sub-list inside a boundary group, plus the empty group (op_table.py:408-417)."""
    out = [[]]
    for sub in groups:
        for length in range(1, len(sub) + 1):
            for start in range(len(sub) - length + 1):
                out.append(list(sub[start:start + length]))
    return out


def get_candidate_operator_groups(context_parallel_size: int = 1):
    (_, _, fwd), (_, _, bwd) = operator_list_prune(context_parallel_size)
    return candidate_groups(fwd), candidate_groups(bwd)
