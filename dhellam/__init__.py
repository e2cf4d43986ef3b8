"""The reference's package name over the MI355X operator path.

``dhellam`` here is a thin re-export of ``dhellam_amd`` under the names the reference's callers import
(dhellam/__init__.py:1-5, setup.py:234-244 builds ``dhellam._Clib``), so that their import lines resolve
unchanged.  What is NOT here is what lies outside the per-rank operator path on one GPU: the collectives
(``dhellam.operators.comm``: the sequence-parallel gather / reduce-scatter are the identity for one rank and
refuse more than one; p2p and chunked collective+GEMM ops raise) and the Megatron adaptor.
"""
from dhellam.operators.layernorm_column import gemm_fwd, gemm_bwd, gemm_fwd_event
from dhellam.operators.layernorm import pylayernorm_fwd, pylayernorm_bwd
from dhellam.operators.comm import gather_along_first_dim, reduce_scatter_along_first_dim
from dhellam._Clib import pymha_varlen_fwd, pymha_varlen_bwd
from dhellam.common.common import _get_qkv_layout
