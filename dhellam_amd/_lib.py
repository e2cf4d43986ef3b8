"""ctypes loader for ``libdhellam_hip.so`` (the C ABI in ``include/dhellam_hip.h``).

PyTorch is used only as the owner of device memory and streams: tensors are
passed down as raw ``data_ptr()`` addresses plus sizes.  There is no fallback:
if the shared object is missing, or a call fails, a ``RuntimeError`` is raised.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libdhellam_hip.so"

DH_F32, DH_BF16, DH_F16 = 0, 1, 2
_DTYPES = {torch.float32: DH_F32, torch.bfloat16: DH_BF16, torch.float16: DH_F16}

_vp, _i64, _i32, _f32, _sz = C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_size_t

# name -> (restype, argtypes); must list every symbol the header declares.
SIGNATURES = {
    "dh_version": (_i32, []),
    "dh_last_error": (C.c_char_p, []),
    "dh_copy_bytes": (_i32, [_vp, _vp, _i64, _vp]),
    "dh_delay": (_i32, [_i64, _vp]),
    "dh_host_delay": (_i32, [_i64, _vp]),
    "dh_comm_proxy_create": (_i32, [_i32, _vp]),
    "dh_comm_proxy_launch": (_i32, [_vp, _i64, _i64, _vp]),
    "dh_comm_proxy_post": (_i32, [_vp, _i32, _vp]),
    "dh_comm_proxy_wait": (_i32, [_vp, _i32, _vp]),
    "dh_comm_proxy_stop": (_i32, [_vp, _vp]),
    "dh_comm_proxy_log": (_i32, [_vp, _i32, _i64, _vp, _vp, _vp]),
    "dh_gemm": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _vp, _sz, _vp]),
    "dh_gemm_tt": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _vp, _sz, _vp]),
    "dh_stream_create_cu_mask": (_i32, [_vp, _i32, _vp]),
    "dh_stream_destroy": (_i32, [_vp]),
    "dh_transpose_2d": (_i32, [_vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp]),
    "dh_cross_entropy_fwd": (_i32, [_vp, _vp, _i64, _i64, _i64, _i64, _f32, _i32, _vp, _vp, _vp, _vp, _vp, _i64, _vp,
                                    _vp, _vp]),
    "dh_cross_entropy_bwd": (_i32, [_vp, _i64, _i32, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _i32, _vp, _i64,
                                    _vp]),
    "dh_embedding_fwd": (_i32, [_vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp, _vp]),
    "dh_embedding_bwd": (_i32, [_vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp, _i32, _vp]),
    "dh_masked_mean_fwd": (_i32, [_vp, _vp, _i64, _f32, _vp, _vp]),
    "dh_masked_mean_bwd": (_i32, [_vp, _vp, _i64, _f32, _vp, _vp]),
    "dh_norm_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _i32, _i32, _vp]),
    "dh_add_norm_fwd": (_i32, [_vp] * 8 + [_i64, _i64, _f32, _i32, _i32, _vp]),
    "dh_norm_bwd_workspace_bytes": (_sz, [_i64, _i64]),
    "dh_norm_bwd": (_i32, [_vp] * 10 + [_sz, _i64, _i64, _i32, _i32, _i32, _vp]),
    "dh_swiglu_fwd": (_i32, [_vp, _vp, _i64, _i64, _i32, _vp]),
    "dh_swiglu_bwd": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32, _vp]),
    "dh_swiglu_bwd_t": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _vp]),
    "dh_swiglu_fwd_t": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32, _vp]),
    "dh_residual_add": (_i32, [_vp, _vp, _vp, _i64, _i32, _vp]),
    "dh_gelu": (_i32, [_vp, _vp, _i64, _i32, _vp]),
    "dh_bias_mask_add": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _vp]),
    "dh_rope": (_i32, [_vp] * 6 + [_i64, _i32, _i32, _i32, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _vp]),
    "dh_attn_fwd": (_i32, [_vp] * 7 + [_i32] * 6 + [_i64] * 4 + [_f32, _i32, _i32, _vp]),
    "dh_attn_bwd_workspace_bytes": (_sz, [_i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32]),
    "dh_attn_bwd_min_workspace_bytes": (_sz, [_i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32]),
    "dh_attn_bwd": (_i32, [_vp] * 11 + [_sz] + [_vp] * 2 + [_i32] * 3 + [_i64] * 2 + [_i32] * 3 + [_i64] * 8 + [_f32, _i32, _i32, _vp]),
    "dh_attn_bwd_set_ds_limit": (None, [_sz]),
    "dh_attn_bwd_set_ds_when_full": (None, [_i32]),
    "dh_attn_bwd_acc": (_i32, [_vp] * 11 + [_sz] + [_vp] * 2 + [_i32] * 3 + [_i64] * 2 + [_i32] * 3 + [_i64] * 8 + [_f32, _i32, _i32, _i32, _vp]),
    "dh_attn_merge": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp]),
    "dh_moe_route_topk": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _vp]),
    "dh_moe_sort_workspace_bytes": (_sz, [_i64, _i32]),
    "dh_moe_sort": (_i32, [_vp] * 6 + [_sz, _i64, _i32, _vp]),
    "dh_moe_sort_static_max_assign": (_i64, []),
    "dh_moe_sort_static": (_i32, [_vp] * 5 + [_i64, _i32, _vp]),
    "dh_moe_gather_rows": (_i32, [_vp] * 5 + [_i32, _i32, _i64, _i32, _i64, _i32, _vp]),
    "dh_moe_scatter_rows": (_i32, [_vp] * 5 + [_i32, _i32, _i64, _i32, _i64, _i32, _vp]),
    "dh_moe_gate_grad": (_i32, [_vp] * 5 + [_i32, _i32, _i64, _i32, _i64, _i32, _vp]),
    "dh_grouped_gemm_workspace_bytes": (_sz, []),
    "dh_grouped_gemm_nt": (_i32, [_vp] * 4 + [_i32, _i64, _i64, _i64, _i32, _vp, _sz, _vp]),
    "dh_grouped_gemm_nn": (_i32, [_vp] * 4 + [_i32, _i64, _i64, _i64, _i32, _vp, _sz, _vp]),
    "dh_grouped_gemm_tn": (_i32, [_vp] * 4 + [_i32, _i64, _i64, _i64, _i32, _i32, _vp]),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared object once and attach the signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m dhellam_amd.build` "
            "(there is no non-HIP fallback)")
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != 0:
        msg = load().dh_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"dhellam_hip error {rc}: {msg}")


def dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {t.dtype}") from None


def ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


def cur_stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def need_cuda(*ts) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("dhellam operators need tensors on the GPU")


def mark_written(*ts) -> None:
    """A kernel of this library is about to write these tensors through their raw pointers, which does not move
    torch's version counter: whatever a producer hung on them that described their OLD contents (the transposed
    twin that the SwiGLU kernels leave for the weight-gradient GEMM) is dropped here."""
    for t in ts:
        if t is not None:
            t.__dict__.pop("_dh_rows_transposed", None)
