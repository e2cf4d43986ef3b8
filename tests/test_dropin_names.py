"""The reference's own import lines resolve against this build (no GPU): its package name ``dhellam`` is shipped as
a re-export of ``dhellam_amd``, so a caller written for the reference imports the same names from the same
modules.  The lines below are the ``from dhellam... import ...`` statements of the reference's package, search
tools and micro-benchmark (dhellam/__init__.py:1-5, dhellam/core/dstb.py:5-14, dhellam/core/dshb.py:16-19,
dhellam/core/dsllm.py:5-9, dhellam/operators/layernorm_column.py:3-4, search/execute.py:7-12,
search/profiler.py:3, micro_benchmark/overlap.py:4-19), minus the Megatron adaptor."""
import inspect

import pytest

REFERENCE_IMPORT_LINES = """
from dhellam.operators.layernorm_column import gemm_fwd,gemm_bwd,gemm_fwd_event
from dhellam.operators.layernorm import pylayernorm_fwd,pylayernorm_bwd
from dhellam.operators.comm import gather_along_first_dim,reduce_scatter_along_first_dim
from dhellam._Clib import pymha_varlen_fwd,pymha_varlen_bwd
from dhellam.common.common import _get_qkv_layout
from dhellam import gemm_fwd,pylayernorm_fwd,gather_along_first_dim,pymha_varlen_fwd,_get_qkv_layout,reduce_scatter_along_first_dim,gemm_fwd_event
from dhellam.operators.bda import bda_fwd,bda_bwd
from dhellam.operators.swiglu import swiglu,swiglu_back
from dhellam.common.common import print_rank0
from dhellam import gemm_bwd,pylayernorm_bwd,gather_along_first_dim,pymha_varlen_bwd,_get_qkv_layout,reduce_scatter_along_first_dim
from dhellam.operators.layernorm_column import dgrad_bwd,wgrad_bwd
from dhellam.common.global_variables import GLOBAL_VARIABLES
from dhellam.operators.ring_attn import fa_cp_block_fwd,fa_cp_block_bwd
from dhellam.common.template_launch import template_fwd_new, template_bwd_new
from dhellam import pylayernorm_fwd,pylayernorm_bwd
from dhellam.core.dshb import DSHB
from dhellam.core.dstb import DSTB
from dhellam._Clib import pygemm as gemm
from dhellam.common.common import get_workspace,print_rank0
from dhellam.core.dstb import DSTB, DCoperation, exec
from dhellam.core.dstb import DCFunc
from dhellam.core.dsllm import DSLLM
from dhellam.common.benchmark import benchmark_ms_ops
from dhellam.common.benchmark import benchmark_ms
from dhellam.operators.comm import gather_along_first_dim, reduce_scatter_along_first_dim, chunk_allgather_gemm, chunk_gemm_reduce_scatter
from dhellam.operators.comm import flash_attn_p2p_communicate
from dhellam._Clib import pymha_varlen_fwd, pymha_varlen_bwd
from dhellam._Clib import pygemm, pygelu, pybda, add_tensors
from dhellam.adaptor.parallel_state import get_tensor_model_parallel_rank, get_tensor_model_parallel_world_size
""".strip().splitlines()


@pytest.mark.parametrize("line", REFERENCE_IMPORT_LINES)
def test_reference_import_line_resolves(line):
    ns = {}
    exec(line, ns)          # noqa: S102 - the line is one of the constants above
    assert len(ns) > 1


WANT_PARAMS = {
    "pygemm": ["inputA", "inputB", "outputD", "input_workspace", "workspaceSize", "transa", "transb",
               "grad_accumulate", "math_sm_count", "profiling"],
    "pygelu": ["input", "output", "profiling"],
    "pybda": ["input", "bias", "residual", "output", "prob", "profiling"],
    "add_tensors": ["a", "b"],
    "pymha_varlen_fwd": ["q", "k", "v", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "p_dropout",
                         "softmax_scale", "is_causal", "return_softmax", "math_sm_count", "profiling"],
    "pymha_varlen_bwd": ["dout", "q", "k", "v", "out", "softmax_lse", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q",
                         "max_seqlen_k", "p_dropout", "softmax_scale", "is_causal", "rng_state", "deterministic",
                         "math_sm_count", "profiling", "stream_ptr"],
}
WANT_RETURNS = {"pygemm": "float", "pygelu": "float", "pybda": "float", "add_tensors": "torch.Tensor",
                "pymha_varlen_fwd": "list[torch.Tensor]", "pymha_varlen_bwd": "list[torch.Tensor]"}


def test_compiled_binding_signatures_are_the_references():
    """``dhellam._Clib`` is the compiled pybind11 extension (csrc/torchapi.cpp:2-9 in the reference): its six
    functions take the positional parameters of csrc/operators/ops.h:18-81, in that order, and return what the
    reference's do.  pybind11 puts the signature into the first line of the docstring."""
    import re
    import dhellam._Clib as C
    assert C.__file__.endswith(".so"), C.__file__
    assert sorted(n for n in dir(C) if not n.startswith("_")) == sorted(WANT_PARAMS)
    for name, params in WANT_PARAMS.items():
        first = getattr(C, name).__doc__.splitlines()[0]
        m = re.fullmatch(rf"{name}\((.*)\) -> (.*)", first)
        assert m, first
        got = [p.split(":")[0].strip() for p in m.group(1).split(", ")]
        assert got == params, (name, got)
        assert m.group(2) == WANT_RETURNS[name], (name, m.group(2))


def test_ctypes_mirror_signatures_are_the_references():
    """The Python mirror of the same module (``dhellam_amd._Clib``, ctypes over the C ABI) keeps the same names."""
    import dhellam_amd._Clib as C
    for name, params in WANT_PARAMS.items():
        got = list(inspect.signature(getattr(C, name)).parameters)
        assert got == params, (name, got)


def test_compiled_binding_refuses_what_the_library_does_not_do():
    """Error paths that need no GPU: they surface as RuntimeError like the reference's TORCH_CHECKs."""
    import torch
    import dhellam._Clib as C
    x = torch.zeros(4, 2, 8)
    cu = torch.tensor([0, 4], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="dropout"):
        C.pymha_varlen_fwd(x, x, x, cu, cu, 4, 4, 0.1, 1.0, True, False, 0, False)
    with pytest.raises(RuntimeError, match="GPU"):
        C.pymha_varlen_fwd(x, x, x, cu, cu, 4, 4, 0.0, 1.0, True, False, 0, False)
    with pytest.raises(RuntimeError, match="TT layout"):
        C.pygemm(x[0], x[0], x[0], x[0], 0, True, True, False, 0, False)
    assert torch.equal(C.add_tensors(torch.ones(3), torch.ones(3)), torch.full((3,), 2.0))


def test_one_rank_collectives_and_refusals():
    import torch
    from dhellam.operators.comm import chunk_allgather_gemm, gather_along_first_dim, reduce_scatter_along_first_dim
    x = torch.arange(6.0).view(3, 2)
    out, handle = gather_along_first_dim(x, gpus=1, comm_group=None, async_op=True)
    assert out is x and handle.wait() is None
    out, handle = reduce_scatter_along_first_dim(x, gpus=1)
    assert out is x and handle is None
    with pytest.raises(RuntimeError):
        gather_along_first_dim(x, gpus=8)
    with pytest.raises(RuntimeError):
        chunk_allgather_gemm(x)
    from dhellam.adaptor.megatron import initialize_dhellam_megatron
    with pytest.raises(RuntimeError):
        initialize_dhellam_megatron()


def test_qkv_layout_names():
    import torch
    from dhellam import _get_qkv_layout
    t, h, d = 6, 4, 8
    packed = torch.zeros(t, 3, h, d)
    assert _get_qkv_layout(packed[:, 0], packed[:, 1], packed[:, 2], "thd")[0] == "t3hd"
    packed = torch.zeros(t, h, 3, d)
    assert _get_qkv_layout(packed[:, :, 0], packed[:, :, 1], packed[:, :, 2], "thd")[0] == "th3d"
    q, kv = torch.zeros(t, h, d), torch.zeros(t, 2, h, d)
    assert _get_qkv_layout(q, kv[:, 0], kv[:, 1], "thd")[0] == "thd_t2hd"
    kv = torch.zeros(t, h, 2, d)
    assert _get_qkv_layout(q, kv[:, :, 0], kv[:, :, 1], "thd")[0] == "thd_th2d"
    assert _get_qkv_layout(q, torch.zeros(t, h, d), torch.zeros(t, h, d), "thd")[0] == "thd_thd_thd"
    with pytest.raises(AssertionError):
        _get_qkv_layout(q.transpose(1, 2), q, q)
