"""Streams bound to a subset of the compute units.

The reference partitions the GPU between its streams with libsmctrl (csrc/operators/smctrl.cpp:135-160,
``math_sm_count`` of pygemm, csrc/operators/ops.h:30).  On MI355X the same thing is a property of the
stream: ``hipExtStreamCreateWithCUMask``.  What it is for here: a library GEMM allocates every register
of every SIMD, so a kernel launched meanwhile on another stream -- however small -- starts only when the
GEMM has placed its last workgroup (a 55 us stand-in for a collective was measured taking 410 us next to
a 370 us GEMM).  Keeping a few compute units out of the compute streams' masks and giving exactly those
to the communication streams removes that wait (59-60 us, every time).  The price: a kernel whose grid
fills 256 compute units a whole number of times (512 GEMM tiles, the attention kernels' 256 workgroups)
needs one more round on 248, so the partition pays off only for grids sized for it.
"""
from __future__ import annotations

import ctypes
from typing import List

import torch

from .. import _lib

N_XCD = 8     # MI355X: 8 XCDs of 32 compute units; bit i of a mask is compute unit i // 8 of XCD i % 8


def cu_mask_words(n_cus: int, first: int, count: int) -> List[int]:
    """Mask words with bits [first, first + count) set, for a device of ``n_cus`` compute units."""
    if not (0 <= first and count > 0 and first + count <= n_cus):
        raise ValueError(f"compute units [{first}, {first + count}) outside a device of {n_cus}")
    words = [0] * ((n_cus + 31) // 32)
    for i in range(first, first + count):
        words[i // 32] |= 1 << (i % 32)
    return words


# ``torch.cuda.ExternalStream`` only borrows a handle.  The library is the owner of last resort: it keeps the
# list of live masked streams and ends those still open in an exit handler that runs after the interpreter has
# shut down and before the HIP runtime's own destructors.  ``_LIVE`` mirrors that list for this module.
_LIVE: set = set()


def _destroy_handle(handle: int) -> None:
    if handle in _LIVE:
        _LIVE.discard(handle)
        _lib.check(_lib.load().dh_stream_destroy(handle))


def stream_with_cu_mask(words: List[int]) -> torch.cuda.Stream:
    arr = (ctypes.c_uint32 * len(words))(*words)
    out = ctypes.c_void_p()
    _lib.check(_lib.load().dh_stream_create_cu_mask(ctypes.cast(arr, ctypes.c_void_p), len(words), ctypes.byref(out)))
    _LIVE.add(out.value)
    return torch.cuda.ExternalStream(out.value)


def destroy_stream(stream: torch.cuda.Stream) -> None:
    """Ends a stream made by ``stream_with_cu_mask`` after waiting for its work.  Drop every tensor that was used
    on the stream first: the caching allocator records an event on each stream a block was used on when the
    block is freed, and a destroyed stream cannot take one.  Streams that are never destroyed by hand are
    destroyed by the library when the process exits."""
    stream.synchronize()
    _destroy_handle(stream.cuda_stream)


class PartitionedStreams:
    """The streams of one partition of the GPU and their owner: unpacks as ``(compute, comm)``, and as a
    context manager (or through ``close()``) ends the streams when the block is left."""

    def __init__(self, compute: List[torch.cuda.Stream], comm: List[torch.cuda.Stream]):
        self.compute, self.comm = compute, comm

    def __iter__(self):
        return iter((self.compute, self.comm))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False

    def close(self) -> None:
        for st in self.compute + self.comm:
            if st.cuda_stream in _LIVE:
                destroy_stream(st)
        self.compute, self.comm = [], []


def partitioned_streams(reserved_per_xcd: int = 1, n_compute: int = 2, n_comm: int = 2) -> PartitionedStreams:
    """(compute streams, communication streams): the communication streams own ``reserved_per_xcd`` compute
    units of every XCD (the highest mask bits), the compute streams all the others.  Use as
    ``with partitioned_streams() as (compute, comm): ...`` so that the streams end with the block."""
    n_cus = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    reserved = reserved_per_xcd * N_XCD
    if not 0 < reserved < n_cus:
        raise ValueError(f"cannot reserve {reserved} of {n_cus} compute units")
    comp = cu_mask_words(n_cus, 0, n_cus - reserved)
    comm = cu_mask_words(n_cus, n_cus - reserved, reserved)
    return PartitionedStreams([stream_with_cu_mask(comp) for _ in range(n_compute)],
                              [stream_with_cu_mask(comm) for _ in range(n_comm)])
