"""The resident communication proxy (``dh_comm_proxy_*``): collectives that a strand posts on its stream and waits
for without a kernel launch per collective.

The reference posts its collectives on a third stream and lets the compute op wait for the handle
(dhellam/core/dstb.py:1142-1188).  A collective that is a kernel of its own cannot start while a large GEMM of the
other strand owns every compute unit; the proxy is one kernel with one resident wavefront per strand, reached through
stream writes and stream waits that the command processor carries out.  On one GPU a request is carried out by
waiting for the duration the collective would take.
"""
from __future__ import annotations

import ctypes
from typing import List, Sequence, Tuple

import torch

from .. import _lib


class CommProxy:
    """``slots`` channels (one per strand).  Use per step::

        proxy.launch(duration_us)                 # on the proxy's own stream
        ...  proxy.collective(slot, stream) ...   # post + wait on the strand's stream, any number of times
        proxy.stop([stream_of_slot_0, stream_of_slot_1])
    """

    def __init__(self, slots: int = 2):
        self.slots = slots
        out = ctypes.c_void_p()
        _lib.check(_lib.load().dh_comm_proxy_create(slots, ctypes.byref(out)))
        self._h = out.value
        self.stream = torch.cuda.Stream()
        self.running = False

    def launch(self, duration_us: float, limit_ms: float = 2000.0) -> None:
        _lib.check(_lib.load().dh_comm_proxy_launch(self._h, int(duration_us * 1000), int(limit_ms * 1e6),
                                                    self.stream.cuda_stream))
        self.running = True

    def collective(self, slot: int, stream: torch.cuda.Stream) -> None:
        """One collective of the slot's strand: posted behind the stream's earlier work, and the stream's later
        work waits until the proxy has carried it out."""
        lib = _lib.load()
        _lib.check(lib.dh_comm_proxy_post(self._h, slot, stream.cuda_stream))
        _lib.check(lib.dh_comm_proxy_wait(self._h, slot, stream.cuda_stream))

    def stop(self, streams: Sequence[torch.cuda.Stream]) -> None:
        """Ends the launch: slot i takes no request after what ``streams[i]`` holds now."""
        assert len(streams) == self.slots
        arr = (ctypes.c_void_p * self.slots)(*[s.cuda_stream for s in streams])
        _lib.check(_lib.load().dh_comm_proxy_stop(self._h, ctypes.cast(arr, ctypes.c_void_p)))
        self.running = False

    def log(self, slot: int, max_entries: int = 256) -> List[Tuple[float, float]]:
        """(start, end) in microseconds (device clock, arbitrary origin) of the collectives the slot carried out in
        the launches since the last call; synchronises the device first."""
        torch.cuda.synchronize()
        a = (ctypes.c_int64 * max_entries)()
        b = (ctypes.c_int64 * max_entries)()
        n = ctypes.c_int64()
        _lib.check(_lib.load().dh_comm_proxy_log(self._h, slot, max_entries, ctypes.cast(a, ctypes.c_void_p),
                                                 ctypes.cast(b, ctypes.c_void_p), ctypes.byref(n)))
        return [(a[i] / 1e3, b[i] / 1e3) for i in range(n.value)]
