"""Small helpers of dhellam/common/common.py that the hot path touches."""
import torch

_workspace = {}


def get_workspace() -> torch.Tensor:
    """GEMM workspace, cached per device (the reference re-allocates 4/32 MiB on every
    call, common.py:7-13); hipBLASLt manages its own, so this is only kept for callers."""
    dev = torch.cuda.current_device()
    if dev not in _workspace:
        _workspace[dev] = torch.empty(4_194_304, dtype=torch.uint8, device=f"cuda:{dev}")
    return _workspace[dev]


def print_rank0(*args) -> None:
    if not torch.distributed.is_available() or not torch.distributed.is_initialized() \
            or torch.distributed.get_rank() == 0:
        print(*args)


def _get_qkv_layout(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, qkv_format: str = "sbhd"):
    """Memory layout of q, k, v as the reference names it (common.py:19-118, TransformerEngine's convention):
    returns (layout, q, k, v).  ``<fmt>`` = sbhd / bshd / thd; layouts: ``..3hd`` / ``..h3d`` (one buffer,
    interleaved before / after the head dim), ``<fmt>_..2hd`` / ``<fmt>_..h2d`` (k and v share a buffer),
    ``<fmt>_<fmt>_<fmt>`` (three buffers).  Tensors that fit none are made contiguous (then three buffers)."""
    if not all(x.stride(-1) == 1 for x in (q, k, v)):
        raise AssertionError("q, k and v must have stride 1 in their last dimension!")

    def classify(q, k, v):
        same = lambda ts, f: all(f(t) == f(ts[0]) for t in ts)
        ptr = lambda t: t.untyped_storage().data_ptr()
        qkv, kv = (q, k, v), (k, v)
        one_qkv = same(qkv, ptr) and same(qkv, lambda t: t.stride()) and same(qkv, lambda t: tuple(t.shape))
        one_kv = same(kv, ptr) and same(kv, lambda t: t.stride()) and same(kv, lambda t: tuple(t.shape))
        d, hd = q.shape[-1], q.shape[-1] * q.shape[-2]
        off = lambda ts, unit: all(i * unit == t.storage_offset() for i, t in enumerate(ts))
        dk, hdk = k.shape[-1], k.shape[-1] * k.shape[-2]
        if one_qkv and off(qkv, hd) and not off(qkv, d):
            return qkv_format[:-2] + "3" + qkv_format[-2:]
        if one_qkv and off(qkv, d):
            return qkv_format[:-1] + "3" + qkv_format[-1:]
        if one_kv and off(kv, hdk) and not off(kv, dk):
            return qkv_format + "_" + qkv_format[:-2] + "2" + qkv_format[-2:]
        if one_kv and off(kv, dk):
            return qkv_format + "_" + qkv_format[:-1] + "2" + qkv_format[-1:]
        if same(kv, lambda t: t.stride()) and same(kv, lambda t: tuple(t.shape)):
            return "_".join([qkv_format] * 3)
        return "not_supported"

    layout = classify(q, k, v)
    if layout == "not_supported":
        q, k, v = (x.contiguous() for x in (q, k, v))
        layout = classify(q, k, v)
    if layout == "not_supported":
        raise Exception("The provided qkv memory layout is not supported!")
    return layout, q, k, v
