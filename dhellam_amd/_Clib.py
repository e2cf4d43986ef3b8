"""Python mirror of the reference's native module ``dhellam._Clib``.

The reference exports six functions from a pybind11 torch extension
(csrc/torchapi.cpp:2-9, signatures csrc/operators/ops.h:18-81).  The same names
with the same positional arguments and return conventions are provided here as
thin shims over the C ABI of ``libdhellam_hip.so``; tensors are only carriers
of device pointers.  Functions the reference does not have (RMSNorm, RoPE,
merge, MoE, grouped GEMM) are exported under ``py*`` names in the same style.
"""
from __future__ import annotations

import ctypes as C
import weakref
from typing import Optional

import torch

from . import _lib

__all__ = ["add_tensors", "pygemm", "dense_gemm", "dense_ok", "keep_transposed", "refresh_transposed", "wgrad_gemm", "wgrad_layout", "pygelu", "pybda", "pymha_varlen_fwd", "pymha_varlen_bwd", "pyattn_merge",
           "pyrmsnorm_fwd", "pyrmsnorm_bwd", "pyrope_fwd", "pyrope_bwd", "pyswiglu_fwd", "pyswiglu_bwd",
           "pymoe_route_topk", "pymoe_sort", "pymoe_permute", "pymoe_unpermute", "pygrouped_gemm_nt",
           "pygrouped_gemm_nn", "pygrouped_gemm_tn", "pycross_entropy_fwd", "pycross_entropy_bwd",
           "pyembedding_fwd", "pyembedding_bwd"]


def _timed(profiling: bool, stream, fn):
    """Run fn(); with ``profiling`` bracket it with events on ``stream`` and return ms
    (the reference brackets with cudaEvent and synchronises only when profiling,
    csrc/operators/gemm.cu:101-131)."""
    if not profiling:
        fn()
        return 0.0
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record(stream)
    fn()
    end.record(stream)
    end.synchronize()
    return float(start.elapsed_time(end))


def add_tensors(a, b):
    """ops.h:67-69."""
    return a + b


GEMM_WORKSPACE_BYTES = 32 << 20
_gemm_ws: dict = {}


def _gemm_workspace(device, stream_ptr: int) -> torch.Tensor:
    """One workspace per (device, stream): kernels that split a product over workgroups keep partial tiles
    there, so two streams must not share one."""
    key = (str(device), stream_ptr)
    ws = _gemm_ws.get(key)
    if ws is None:
        ws = torch.empty(GEMM_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
        _gemm_ws[key] = ws
    return ws


def dense_ok(*tensors) -> bool:
    """True when ``dh_gemm`` takes these operands as they are: 2-D, contiguous, on the GPU."""
    return all(t.is_cuda and t.dim() == 2 and t.is_contiguous() for t in tensors)


def dense_gemm(A, B, D, transa: bool, transb: bool, accumulate: bool, workspace=None, workspace_bytes: int = 0) -> None:
    """``dh_gemm`` on the current stream, in the reference's operand convention (see ``pygemm``)."""
    if not dense_ok(A, B, D):
        raise RuntimeError("dense_gemm: operands must be contiguous 2-D GPU tensors")
    if A.dtype != B.dtype or D.dtype not in (A.dtype, torch.float32):
        raise RuntimeError(f"dense_gemm: operand types {A.dtype}, {B.dtype} -> {D.dtype} not supported")
    m = A.shape[0] if transa else A.shape[1]
    n = B.shape[1] if transb else B.shape[0]
    if tuple(D.shape) != (n, m):
        raise RuntimeError(f"dense_gemm: output is {tuple(D.shape)}, the product is {(n, m)}")
    stream = torch.cuda.current_stream()
    _lib.mark_written(D)
    if workspace is None or not getattr(workspace, "is_cuda", False) or workspace_bytes <= 0:
        workspace = _gemm_workspace(A.device, stream.cuda_stream)
        workspace_bytes = workspace.numel()
    elif workspace.numel() * workspace.element_size() < workspace_bytes:
        raise RuntimeError("dense_gemm: workspace tensor smaller than workspaceSize")
    if (transa and A.shape[1] == 0) or (not transa and A.shape[0] == 0):
        if not accumulate:
            D.zero_()
        return
    if transa and transb:      # refused by dh_gemm as by the reference's cublas_gemm; the library's own entry for it
        _lib.check(_lib.load().dh_gemm_tt(A.data_ptr(), B.data_ptr(), D.data_ptr(), A.shape[0], A.shape[1], B.shape[0],
                                          B.shape[1], int(accumulate), _lib.dt(A), _lib.dt(D), workspace.data_ptr(),
                                          workspace_bytes, stream.cuda_stream))
        return
    _lib.check(_lib.load().dh_gemm(A.data_ptr(), B.data_ptr(), D.data_ptr(), A.shape[0], A.shape[1], B.shape[0],
                                   B.shape[1], int(transa), int(transb), int(accumulate), _lib.dt(A), _lib.dt(D),
                                   workspace.data_ptr(), workspace_bytes, stream.cuda_stream))


def pygemm(inputA, inputB, outputD, input_workspace, workspaceSize, transa, transb, grad_accumulate, math_sm_count,
           profiling):
    """csrc/operators/gemm.cu:3-170.  Column-major cuBLASLt convention of the reference:
    with row-major tensors A [m?,k?], B, the result is D = op(B) @ op(A) written into
    ``outputD`` (accumulated when ``grad_accumulate``), i.e.

        transa  transb   D
        True    False    B   @ A.T     ("TN": input @ weight.T)
        False   False    B   @ A       ("NN": dgrad)
        False   True     B.T @ A       ("NT": wgrad)

    The product is ``dh_gemm`` (hipBLASLt behind the C ABI).  ``input_workspace`` / ``workspaceSize`` are
    used when given (a GPU tensor of at least that many bytes), otherwise a per-stream 32 MiB buffer.
    ``math_sm_count`` > 0 confines the product to that many compute units, as the reference's libsmctrl
    mask does (csrc/operators/gemm.cu:66-70, smctrl.cpp:135-160): it runs on a stream created with that
    compute-unit mask (cached per device and count), ordered after and before the current stream by events;
    a count above the device's compute units is refused.  For the weight gradient, the smaller operand is
    materialised transposed first where that makes the product faster by more than it costs (``wgrad_layout``).
    """
    _lib.need_cuda(inputA, inputB, outputD)
    stream = torch.cuda.current_stream()
    ws_bytes = int(workspaceSize or 0)

    if transa and transb:
        raise RuntimeError("pygemm: TT layout not allowed")     # as the reference (csrc/operators/gemm.cu)

    def product():
        if transb and not transa:
            wgrad_gemm(inputB, inputA, outputD, grad_accumulate, input_workspace, ws_bytes)
        else:
            dense_gemm(inputA, inputB, outputD, transa, transb, grad_accumulate, input_workspace, ws_bytes)

    return _timed(profiling, stream, lambda: _confined(stream, math_sm_count, lambda st: product()))


_masked_streams: dict = {}


def _masked_stream(count: int) -> torch.cuda.Stream:
    """The stream that owns ``|count|`` compute units of the current device: the first ones for a positive
    count, the last ones for a negative count (the reference's ``reverse``, gemm.cu:20-21).  Mask bits are spread
    over the XCDs round-robin, so the units are shared evenly between them."""
    from .common.streams import cu_mask_words, stream_with_cu_mask
    dev = torch.cuda.current_device()
    n_cus = torch.cuda.get_device_properties(dev).multi_processor_count
    n = abs(count)
    if not 0 < n <= n_cus:
        raise RuntimeError(f"math_sm_count={count} outside the {n_cus} compute units of this device")
    key = (dev, count)
    if key not in _masked_streams:
        _masked_streams[key] = stream_with_cu_mask(cu_mask_words(n_cus, 0 if count > 0 else n_cus - n, n))
    return _masked_streams[key]


def _confined(stream, math_sm_count, launch):
    """``launch(stream_to_use)`` on ``stream``, or -- with a non-zero ``math_sm_count`` -- on the masked stream of
    that many compute units, ordered after and before ``stream`` by events (the MI355X form of the reference's
    per-launch libsmctrl mask, csrc/operators/smctrl.cpp:135-160)."""
    math_sm_count = int(math_sm_count or 0)
    if math_sm_count == 0:
        return launch(stream)
    masked = _masked_stream(math_sm_count)
    masked.wait_stream(stream)
    with torch.cuda.stream(masked):
        res = launch(masked)
    stream.wait_stream(masked)
    return res


def transpose_2d(src: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row-major [rows, cols] -> row-major [cols, rows] (16-bit elements) on the current stream."""
    _lib.need_cuda(src)
    if not (src.dim() == 2 and src.stride(1) == 1):
        raise RuntimeError("transpose_2d: src must be 2-D with unit inner stride")
    rows, cols = src.shape
    if out is None:
        out = torch.empty((cols, rows), dtype=src.dtype, device=src.device)
    elif not (out.shape == (cols, rows) and out.stride(1) == 1 and out.dtype == src.dtype):
        raise RuntimeError("transpose_2d: out must be [cols, rows] of src's dtype with unit inner stride")
    _lib.check(_lib.load().dh_transpose_2d(src.data_ptr(), out.data_ptr(), rows, cols, src.stride(0), out.stride(0),
                                           _lib.dt(src), torch.cuda.current_stream().cuda_stream))
    return out


# The weight-gradient product dW[N, K] = dY[T, N]^T X[T, K] reads both operands along their strided dimension, the
# GEMM library's slowest layout here.  Measured at T = 4096, bf16, accumulating (us; N, K = 7168, 8192 / 8192, 3584 /
# 1280, 8192 / 8192, 1024):   as given 464 / 233 / 105 / 85;   dY^T row-major 380 / 190 / 87 / 72;   X^T row-major
# (the layout ``dh_gemm`` refuses, ``dh_gemm_tt``) 383 / 188 / 95 / 70;   both row-major (the forward's layout)
# 335 / 165 / 76 / 61.  One transposed operand is worth 15-20 % whichever it is, so the SMALLER one is transposed
# (dh_transpose_2d moves 5.5-6 TB/s: [4096, 8192] in 24 us, [4096, 3584] in 11 us, [4096, 1024] in 8 us): X when the
# weight has fewer inputs than outputs (fc2, the attention output projection, the vocabulary projection), dY
# otherwise (qkv, fc1 -- where the kernel that produces dY writes the transpose alongside).  Both transposed would
# be faster still, but for that layout the library picks a kernel that splits tiles over workgroups, and its
# accumulation into dW does not always give the same bits when another kernel shares the GPU (1 step in 40-100
# of the double-strand schedule differed from the serial one in the last bits of one weight gradient; giving each
# stream its own workspace does not change that), while the two schedules are required to agree bit for bit: not
# used.
WGRAD_TRANSPOSE_GRAD_MIN_K = 3072
WGRAD_TRANSPOSE_MIN_ELEMS = 1 << 20


def _can_transpose(t: torch.Tensor) -> bool:
    return (t.dtype in (torch.bfloat16, torch.float16) and t.dim() == 2 and t.is_contiguous()
            and t.shape[0] % 8 == 0 and t.shape[1] % 8 == 0 and t.data_ptr() % 16 == 0)


def wgrad_layout(grad: torch.Tensor, data: torch.Tensor) -> str:
    """Which operand of dW = dY^T X is materialised transposed before the library call: "NT" (none), "NN" (dY^T)
    or "TT" (X^T)."""
    (t, n), k = grad.shape, data.shape[1]
    if grad.dtype != data.dtype:
        return "NT"
    if k < n and t * k >= WGRAD_TRANSPOSE_MIN_ELEMS and _can_transpose(data) and _can_transpose(grad):
        return "TT"
    if k >= WGRAD_TRANSPOSE_GRAD_MIN_K and t * n >= WGRAD_TRANSPOSE_MIN_ELEMS and _can_transpose(grad):
        return "NN"
    return "NT"


def wgrad_operands(grad: torch.Tensor, data: torch.Tensor):
    """(lhs, rhs) with lhs @ rhs = grad^T @ data for grad = dY [T, N], data = X [T, K]: the strided view of dY,
    or its materialised row-major transpose where ``wgrad_layout`` says "NN" (a product through torch has no use
    for X^T)."""
    if wgrad_layout(grad, data) == "NN":
        return transpose_2d(grad), data
    return grad.t(), data


def wgrad_gemm(grad: torch.Tensor, data: torch.Tensor, out: torch.Tensor, accumulate: bool, workspace=None,
               workspace_bytes: int = 0) -> None:
    """out [N, K] (+)= grad [T, N]^T @ data [T, K] through the GEMM library, in the layout ``wgrad_layout`` picks."""
    layout = wgrad_layout(grad, data)
    if layout == "NN":
        # the kernel that produced ``grad`` may have left its transpose on it, stamped with the tensor's version
        version, gt = getattr(grad, "_dh_rows_transposed", None) or (None, None)
        if (gt is None or version != grad._version or gt.shape != (grad.shape[1], grad.shape[0])
                or gt.dtype != grad.dtype):
            gt = transpose_2d(grad)
        dense_gemm(data, gt, out, False, False, accumulate, workspace, workspace_bytes)
    elif layout == "TT":
        version, xt = getattr(data, "_dh_rows_transposed", None) or (None, None)
        if (xt is None or version != data._version or xt.shape != (data.shape[1], data.shape[0])
                or xt.dtype != data.dtype):
            xt = transpose_2d(data)
        dense_gemm(xt, grad, out, True, True, accumulate, workspace, workspace_bytes)
    else:
        dense_gemm(data, grad, out, False, True, accumulate, workspace, workspace_bytes)


# The data-gradient product dX[T, K] = dY[T, N] W[N, K] reads the weight along its strided dimension ("NN").  With
# the weight's transpose W^T [K, N] at hand the same product is the forward's layout ("TN": both operands read along
# k), for which the GEMM library has its fastest kernels here: at T = 4096, bf16 (us, NN -> TN; N, K = 1280, 8192 /
# 8192, 1024 / 7168, 8192 / 8192, 3584)  90 -> 72 / 94 -> 73 / 366 -> 308 / 205 -> 174, results identical bit for
# bit.  A weight changes once per optimizer step and is read by every micro-batch's backward in between, and the
# transposes (9 / 7 / 38 / 20 us) cost less than one micro-batch saves, so a weight may be registered to be kept in
# both layouts.  The copy lives on the tensor object.  Who keeps it current: the containers that run a step
# (``LayerRunner.run_*``, ``DSLLMStep.step``, ``run_microbatches``) rebuild the copies of their weights at the START
# of every step with ``refresh_transposed`` -- unconditionally, because the writers that matter do not announce
# themselves: ``p.data.copy_()`` / ``p.data.add_()`` (Megatron's fp16 and distributed optimizers), collectives and raw
# kernels writing into a parameter buffer all leave the tensor's version counter where it was.  In between, a moved
# version counter (any in-place torch op on the tensor itself) also triggers a rebuild at the next use.  A caller
# that drives ``dgrad_gemm`` by hand and updates weights around the counter calls ``refresh_transposed`` itself;
# weights that were never registered take the NN product as before.
_kept_weights: dict = {}        # id(weight) -> weak reference (tensors compare elementwise: no set of them)


def _register_kept(weight: torch.Tensor) -> None:
    key = id(weight)
    if key not in _kept_weights:
        _kept_weights[key] = weakref.ref(weight, lambda _r, key=key: _kept_weights.pop(key, None))


class _Held:
    """What a registered weight carries: the transpose, the version it was built from, the event and stream of
    the build, and one event per stream that has read the copy since (a rebuild waits for them)."""
    __slots__ = ("version", "wt", "built", "stream_ptr", "readers")

    def __init__(self, version, wt, built, stream_ptr):
        self.version, self.wt, self.built, self.stream_ptr, self.readers = version, wt, built, stream_ptr, {}


def keep_transposed(weight: torch.Tensor, refresh: bool = False) -> Optional[torch.Tensor]:
    """Registers ``weight`` [N, K] (or a stack of them, [G, N, K]: the experts of a rank) for a resident transpose
    [K, N] ([G, K, N]) built now, on the current stream, and returns it; None if the tensor is not one
    ``dh_transpose_2d`` takes (then nothing is registered).  ``refresh`` rebuilds the copy of a weight that is
    already registered even if its version counter has not moved; the rebuild writes into the same buffer after
    waiting for every stream that read the old copy."""
    if not (weight.is_cuda and weight.dim() in (2, 3) and weight.is_contiguous() and _can_transpose(weight[0] if weight.dim() == 3 else weight)):
        return None
    held = getattr(weight, "_dh_transposed", None)
    if held is not None and not refresh and held.version == weight._version:
        return held.wt
    stream = torch.cuda.current_stream()
    if held is not None:
        for ptr, ev in held.readers.items():          # the old copy may still be read on another stream
            if ptr != stream.cuda_stream:
                stream.wait_event(ev)
        if held.stream_ptr != stream.cuda_stream:
            stream.wait_event(held.built)
    with torch.no_grad():
        w = weight.detach()
        if w.dim() == 2:
            wt = transpose_2d(w, held.wt if held is not None else None)
        else:
            wt = held.wt if held is not None else torch.empty((w.shape[0], w.shape[2], w.shape[1]), dtype=w.dtype, device=w.device)
            for g in range(w.shape[0]):
                transpose_2d(w[g], wt[g])
    ev = torch.cuda.Event()
    ev.record(stream)
    weight._dh_transposed = _Held(weight._version, wt, ev, stream.cuda_stream)
    _register_kept(weight)
    return wt


def refresh_transposed(weights=None) -> int:
    """Rebuilds the resident transposes of ``weights`` (default: every registered weight still alive) on the current
    stream, whatever their version counters say: the call that follows an optimizer step.  Unregistered tensors in
    ``weights`` are skipped.  Returns how many copies were rebuilt."""
    n = 0
    for w in ([r() for r in list(_kept_weights.values())] if weights is None else weights):
        if isinstance(w, torch.Tensor) and getattr(w, "_dh_transposed", None) is not None:
            keep_transposed(w, refresh=True)
            n += 1
    return n


def transposed_of(weight: torch.Tensor) -> Optional[torch.Tensor]:
    """The resident transpose of a registered weight, brought up to date and safe to read on the current stream;
    None for a weight that was not registered with ``keep_transposed``.  The reader calls ``_note_read`` after
    it has queued its work."""
    held = getattr(weight, "_dh_transposed", None)
    if held is None:
        return None
    if held.version != weight._version:
        return keep_transposed(weight, refresh=True)
    stream = torch.cuda.current_stream()
    if held.stream_ptr != stream.cuda_stream:
        stream.wait_event(held.built)
    return held.wt


def _note_read(weight: torch.Tensor) -> None:
    """Marks the point on the current stream up to which the resident transpose of ``weight`` is being read."""
    held = getattr(weight, "_dh_transposed", None)
    if held is None:
        return
    stream = torch.cuda.current_stream()
    if stream.cuda_stream == held.stream_ptr:
        return                                        # same stream as the builder: already ordered
    ev = held.readers.get(stream.cuda_stream)
    if ev is None:
        ev = held.readers[stream.cuda_stream] = torch.cuda.Event()
    ev.record(stream)


def dgrad_gemm(grad: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> None:
    """out [T, K] = grad [T, N] @ weight [N, K] through ``dh_gemm``: in the forward's layout against the resident
    transpose when the weight has one, else as given."""
    wt = transposed_of(weight)
    if wt is not None and wt.dtype == grad.dtype:
        dense_gemm(wt, grad, out, True, False, False)
        _note_read(weight)
    else:
        dense_gemm(weight, grad, out, False, False, False)


def pygelu(input, output, profiling):
    """csrc/operators/gelu.cu:17-43 (tanh-approximation GELU into ``output``)."""
    _lib.need_cuda(input, output)
    assert input.is_contiguous() and output.is_contiguous() and input.numel() == output.numel()
    lib = _lib.load()
    stream = torch.cuda.current_stream()
    return _timed(profiling, stream, lambda: _lib.check(
        lib.dh_gelu(input.data_ptr(), output.data_ptr(), input.numel(), _lib.dt(input), stream.cuda_stream)))


def pybda(input, bias, residual, output, prob, profiling):
    """csrc/operators/bda.cu:18-62: output = mask * (input + bias) + residual.  Only
    prob = 0 (mask of ones) is implemented; the reference draws its mask with
    torch::dropout."""
    if prob != 0.0:
        raise RuntimeError("pybda: only prob = 0 is implemented")
    _lib.need_cuda(input, bias, residual, output)
    lib = _lib.load()
    stream = torch.cuda.current_stream()
    return _timed(profiling, stream, lambda: _lib.check(
        lib.dh_bias_mask_add(input.data_ptr(), bias.data_ptr(), residual.data_ptr(), None, output.data_ptr(),
                             input.numel(), _lib.dt(input), stream.cuda_stream)))


# ---------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------
def _tok_stride(t: torch.Tensor) -> int:
    if not (t.dim() == 3 and t.stride(2) == 1 and t.stride(1) == t.shape[2]):
        raise RuntimeError("attention tensors must be [tokens, heads, d] with contiguous (heads, d)")
    return t.stride(0)


def _attn_fwd_raw(q, k, v, out, lse, cu_q, cu_k, max_q, max_k, scale, causal, stream_ptr):
    lib = _lib.load()
    _lib.check(lib.dh_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                               cu_q.data_ptr(), cu_k.data_ptr(), cu_q.numel() - 1, int(max_q), int(max_k),
                               q.shape[1], k.shape[1], q.shape[2], _tok_stride(q), _tok_stride(k), _tok_stride(v),
                               _tok_stride(out), float(scale), int(bool(causal)), _lib.dt(q), stream_ptr))


HEAD_DIMS_16BIT = (64, 96, 128, 192, 256)      # head dims the 16-bit kernels are compiled for


def _pad_head_dim(t: torch.Tensor, d_to: int) -> torch.Tensor:
    """``t`` [tokens, heads, d] with zero columns appended up to ``d_to`` (the reference pads the head dim to a
    multiple of 8 the same way, csrc/operators/flash_atten.cu:303-312: zero columns change neither the scores nor the
    first d columns of the result)."""
    d = t.shape[-1]
    if d == d_to:
        return t
    out = t.new_zeros(t.shape[0], t.shape[1], d_to)
    out[..., :d] = t
    return out


def _kernel_head_dim(t: torch.Tensor) -> int:
    """The head dim the kernels run ``t`` at: its own for fp32 and for the compiled 16-bit sizes, else the next
    compiled size (d <= 256 as in the reference, flash_atten.cu:284)."""
    d = t.shape[-1]
    if t.dtype == torch.float32 or d in HEAD_DIMS_16BIT:
        return d
    for s_ in HEAD_DIMS_16BIT:
        if d < s_:
            return s_
    raise RuntimeError(f"attention supports head dims up to 256 (got {d})")


_rng_zero: dict = {}


def _zero_rng_state(device) -> torch.Tensor:
    """The int64[2] seed/offset slot of the return list; always zero (no dropout), one per device."""
    t = _rng_zero.get(device)
    if t is None:
        t = torch.zeros(2, dtype=torch.int64, device=device)
        _rng_zero[device] = t
    return t


def pymha_varlen_fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
                     is_causal, return_softmax, math_sm_count, profiling):
    """ops.h:18-32 / flash_atten.cu:436-477.  Runs on the current stream (``math_sm_count`` != 0: confined to
    that many compute units, see ``_confined``).

    Returns [out, q, k, v, out, softmax_lse, p, rng_state] (+ a CPU fp32 [1] tensor of
    milliseconds when ``profiling``), positions as in flash_atten.cu:429-433.  The
    reference pads the head dim to a multiple of 8 and returns the padded tensors; the
    supported head dims need no padding, so the inputs themselves are returned.
    ``p`` is an empty tensor (return_softmax is only meaningful with dropout) and
    ``rng_state`` is a zero int64[2].  Dropout is not implemented: p_dropout must be 0.
    """
    if p_dropout != 0.0:
        raise RuntimeError("pymha_varlen_fwd: dropout is not implemented (p_dropout must be 0)")
    if return_softmax:
        raise RuntimeError("pymha_varlen_fwd: return_softmax is only supported with dropout in the reference")
    _lib.need_cuda(q, k, v, cu_seqlens_q, cu_seqlens_k)
    if cu_seqlens_q.dtype != torch.int32 or cu_seqlens_k.dtype != torch.int32:
        raise RuntimeError("cu_seqlens must be int32")
    stream = torch.cuda.current_stream()
    b = cu_seqlens_q.numel() - 1
    d, dk_ = q.shape[-1], _kernel_head_dim(q)
    if dk_ != d:        # the padded tensors are what the "padded" slots of the return list hold (flash_atten.cu:429-433)
        q, k, v = _pad_head_dim(q, dk_), _pad_head_dim(k, dk_), _pad_head_dim(v, dk_)
    out_padded = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty((b, q.shape[1], int(max_seqlen_q)), dtype=torch.float32, device=q.device)
    ms = _timed(profiling, stream, lambda: _confined(stream, math_sm_count, lambda st: _attn_fwd_raw(
        q, k, v, out_padded, lse, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, is_causal,
        st.cuda_stream)))
    out = out_padded if dk_ == d else out_padded[..., :d]
    p = torch.empty(0, dtype=q.dtype, device=q.device)
    res = [out, q, k, v, out_padded, lse, p, _zero_rng_state(q.device)]
    if profiling:
        res.append(torch.tensor([ms], dtype=torch.float32))
    return res


_bwd_ws: dict = {}


ATTN_BWD_DS_LIMIT_DEFAULT = 1280 << 20


def set_attn_bwd_ds_limit(nbytes: int = ATTN_BWD_DS_LIMIT_DEFAULT) -> None:
    """Bytes of dS up to which the attention backward keeps dS for its dQ product (``dh_attn_bwd_set_ds_limit``;
    0: always recompute).  Process-wide; it steers the sizing call and the choice inside the backward, which also
    checks the size of the workspace it was handed."""
    _lib.load().dh_attn_bwd_set_ds_limit(int(nbytes))


def _attn_bwd_workspace(nbytes: int, device, stream_ptr: int) -> torch.Tensor:
    key = (str(device), stream_ptr)
    ws = _bwd_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _bwd_ws[key] = ws
    return ws


def _attn_bwd_raw(dout, q, k, v, out, lse, dq, dk, dv, delta, cu_q, cu_k, max_q, max_k, scale, causal, stream_ptr,
                  accumulate_dq=False):
    """``dh_attn_bwd``; with ``accumulate_dq`` the call's dq is added to the contents of ``dq`` inside the kernel."""
    lib = _lib.load()
    b = cu_q.numel() - 1
    nbytes = lib.dh_attn_bwd_workspace_bytes(q.shape[0], k.shape[0], b, int(max_q), q.shape[1], k.shape[1],
                                             q.shape[2], _lib.dt(q))
    ws = _attn_bwd_workspace(nbytes, q.device, stream_ptr)
    _lib.check(lib.dh_attn_bwd_acc(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                   lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), _lib.ptr(delta),
                                   ws.data_ptr(), ws.numel(), cu_q.data_ptr(), cu_k.data_ptr(), b, int(max_q), int(max_k),
                                   q.shape[0], k.shape[0], q.shape[1], k.shape[1], q.shape[2], _tok_stride(q),
                                   _tok_stride(k), _tok_stride(v), _tok_stride(out), _tok_stride(dout),
                                   _tok_stride(dq), _tok_stride(dk), _tok_stride(dv), float(scale), int(bool(causal)),
                                   int(bool(accumulate_dq)), _lib.dt(q), stream_ptr))


def pymha_varlen_bwd(dout, q, k, v, out, softmax_lse, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                     p_dropout, softmax_scale, is_causal, rng_state, deterministic, math_sm_count, profiling,
                     stream_ptr):
    """ops.h:34-52 / flash_atten.cu:760-813.  Unlike the forward it launches on the raw
    stream handle ``stream_ptr`` (flash_atten.cu:784).  Returns [dq, dk, dv, softmax_d]
    (+ CPU ms tensor when profiling).  The result is deterministic regardless of
    ``deterministic`` (no floating-point atomics are used)."""
    if p_dropout != 0.0:
        raise RuntimeError("pymha_varlen_bwd: dropout is not implemented (p_dropout must be 0)")
    _lib.need_cuda(dout, q, k, v, out, softmax_lse)
    b = cu_seqlens_q.numel() - 1
    ext = torch.cuda.ExternalStream(stream_ptr) if stream_ptr else torch.cuda.default_stream()
    with torch.cuda.stream(ext):
        d, dk_ = q.shape[-1], _kernel_head_dim(q)
        if dk_ != d:    # zero columns up to a compiled head dim, as flash_atten.cu:560-575 pads to a multiple of 8
            dout, q, k, v, out = (_pad_head_dim(t, dk_) for t in (dout, q, k, v, out))
        dq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        dk = torch.empty(k.shape, dtype=k.dtype, device=k.device)
        dv = torch.empty(v.shape, dtype=v.dtype, device=v.device)
        softmax_d = torch.zeros((b, q.shape[1], int(max_seqlen_q)), dtype=torch.float32, device=q.device)
        ms = _timed(profiling, ext, lambda: _confined(ext, math_sm_count, lambda st: _attn_bwd_raw(
            dout, q, k, v, out, softmax_lse, dq, dk, dv, softmax_d, cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
            max_seqlen_k, softmax_scale, is_causal, int(st.cuda_stream))))
        if dk_ != d:
            dq, dk, dv = dq[..., :d].contiguous(), dk[..., :d].contiguous(), dv[..., :d].contiguous()
    res = [dq, dk, dv, softmax_d]
    if profiling:
        res.append(torch.tensor([ms], dtype=torch.float32))
    return res


def pyattn_merge(outs, lses, row_begin, rows, out, lse):
    """Fused merge of ring-attention partial results (dhellam/operators/ring_attn.py:26-40
    applied as in :146-195) on the current stream.  outs[s] [b*rows[s], hq, d], lses[s]
    fp32 [b, hq, rows[s]]; out [b*sq, hq, d]; lse fp32 [b, hq, sq]."""
    lib = _lib.load()
    n = len(outs)
    b, hq, sq = lse.shape
    d = out.shape[-1]
    po = (C.c_void_p * n)(*[o.data_ptr() for o in outs])
    pl = (C.c_void_p * n)(*[l.data_ptr() for l in lses])
    rb = (C.c_int32 * n)(*[int(x) for x in row_begin])
    rr = (C.c_int32 * n)(*[int(x) for x in rows])
    for s in range(n):
        assert outs[s].is_contiguous() and lses[s].is_contiguous() and lses[s].dtype == torch.float32
        assert outs[s].shape == (b * rows[s], hq, d) and lses[s].shape == (b, hq, rows[s])
    assert out.is_contiguous() and lse.is_contiguous()
    _lib.check(lib.dh_attn_merge(C.cast(po, C.c_void_p), C.cast(pl, C.c_void_p), C.cast(rb, C.c_void_p),
                                 C.cast(rr, C.c_void_p), n, out.data_ptr(), lse.data_ptr(), b, sq, hq, d,
                                 _lib.dt(out), torch.cuda.current_stream().cuda_stream))


# ---------------------------------------------------------------------------------------
# Binding-level names for the operators the reference does not have (RMSNorm, RoPE, SwiGLU as a
# kernel, MoE, grouped GEMM, the head block).  Same conventions as the six names above: positional
# arguments, work on the current stream, a trailing ``profiling`` flag; results come back as a list
# with the elapsed milliseconds appended when profiling.  They forward to ``dhellam_amd.operators``
# (imported lazily: that package imports this module).
# ---------------------------------------------------------------------------------------
def _ret(values, ms, profiling):
    values = list(values)
    return values + [ms] if profiling else values


def pyrmsnorm_fwd(inp, weight, eps, profiling=False):
    """-> [out, rsigma]"""
    from .operators.layernorm import pylayernorm_fwd
    out, _, rsigma, ms = pylayernorm_fwd(inp, weight, None, eps, 0, False, None, profiling)
    return _ret((out, rsigma), ms, profiling)


def pyrmsnorm_bwd(dout, inp, rsigma, weight, profiling=False):
    """-> [dinp, dweight]"""
    from .operators.layernorm import pylayernorm_bwd
    dinp, dweight, _, ms = pylayernorm_bwd(dout, inp, None, rsigma, weight, 0, False, None, profiling)
    return _ret((dinp, dweight), ms, profiling)


def pyrope_fwd(q, k, positions, theta, profiling=False):
    """-> [q_rot, k_rot]; positions None = 0..T-1"""
    from .operators.rope import rope_fwd
    qr, kr, ms = rope_fwd(q, k, positions, theta, None, None, profiling)
    return _ret((qr, kr), ms, profiling)


def pyrope_bwd(dq, dk, positions, theta, profiling=False):
    from .operators.rope import rope_bwd
    a, b, ms = rope_bwd(dq, dk, positions, theta, None, None, profiling)
    return _ret((a, b), ms, profiling)


def pyswiglu_fwd(y, profiling=False):
    from .operators.swiglu import swiglu
    out, ms = swiglu(y, None, profiling)
    return _ret((out,), ms, profiling)


def pyswiglu_bwd(g, y, profiling=False):
    from .operators.swiglu import swiglu_back
    dy, ms = swiglu_back(g, y, None, None, profiling)
    return _ret((dy,), ms, profiling)


def pymoe_route_topk(logits, k, profiling=False):
    """-> [topk_idx int32 [T, k], gates fp32 [T, k]]"""
    from .operators.moe import route_topk
    idx, gates, ms = route_topk(logits, k, None, profiling)
    return _ret((idx, gates), ms, profiling)


def pymoe_sort(topk_idx, num_experts, profiling=False):
    """-> [plan] (sorted assignment order, destination rows, tokens per expert, expert offsets)"""
    from .operators.moe import sort_assignments
    plan, ms = sort_assignments(topk_idx, num_experts, None, profiling)
    return _ret((plan,), ms, profiling)


def pymoe_permute(x, plan, e_lo, e_hi, max_rows, profiling=False):
    from .operators.moe import permute_fwd
    xp, ms = permute_fwd(x, plan, e_lo, e_hi, max_rows, None, profiling)
    return _ret((xp,), ms, profiling)


def pymoe_unpermute(y, plan, gates, e_lo, e_hi, profiling=False):
    from .operators.moe import unpermute_fwd
    out, ms = unpermute_fwd(y, plan, gates, e_lo, e_hi, None, profiling)
    return _ret((out,), ms, profiling)


def pygrouped_gemm_nt(a, b, offs, out=None):
    from .operators.moe import grouped_gemm_nt
    return grouped_gemm_nt(a, b, offs, None, out)


def pygrouped_gemm_nn(a, b, offs, out=None):
    from .operators.moe import grouped_gemm_nn
    return grouped_gemm_nn(a, b, offs, None, out)


def pygrouped_gemm_tn(a, b, offs, out=None, accumulate=False):
    from .operators.moe import grouped_gemm_tn
    return grouped_gemm_tn(a, b, offs, out, accumulate)


def pycross_entropy_fwd(vocab_parallel_logits, target, label_smoothing=0.0, keep_softmax=True):
    """-> the reference's output dict (dhellam/operators/loss.py:91-97)"""
    from .operators.loss import cross_entropy_fwd
    return cross_entropy_fwd({"vocab_parallel_logits": vocab_parallel_logits, "target": target}, label_smoothing,
                             keep_softmax)


def pycross_entropy_bwd(vocab_parallel_logits, target, fwd_out, dout, grad_out=None):
    from .operators.loss import cross_entropy_bwd
    return cross_entropy_bwd([{"vocab_parallel_logits": vocab_parallel_logits, "target": target}, fwd_out], dout,
                             grad_out)


def pyembedding_fwd(vocab, token_ids):
    from .operators.embedding import word_embedding_fwd
    return word_embedding_fwd({"vocab": vocab, "token_ids": token_ids})["word_embeddings"]


def pyembedding_bwd(vocab, token_ids, dout):
    from .operators.embedding import word_embedding_bwd
    return word_embedding_bwd([{"vocab": vocab, "token_ids": token_ids}, None], dout)
