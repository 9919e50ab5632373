"""Pinned host memory for the small copies of a step (its tables up, the sampled tokens down), allocated once and
used again: allocating pinned memory is a call into the driver that takes as long as a small step's whole launch."""
from __future__ import annotations

from typing import List, Tuple

import numpy as np
import torch


class PinnedPool:
    """int32 pinned buffers. ``upload`` copies a host array to the device through one of them and takes the buffer
    back by itself once the copy has happened; ``acquire`` / ``release`` hand one out for a copy from the device."""

    def __init__(self):
        self._free: List[torch.Tensor] = []
        self._in_flight: List[Tuple[torch.Tensor, "torch.cuda.Event"]] = []

    def _reclaim(self) -> None:
        still = []
        for buf, ev in self._in_flight:
            if ev.query():
                self._free.append(buf)
            else:
                still.append((buf, ev))
        self._in_flight = still

    def acquire(self, n: int) -> torch.Tensor:
        """A pinned int32 buffer of at least ``n`` elements."""
        self._reclaim()
        best = None
        for i, buf in enumerate(self._free):
            if buf.numel() >= n and (best is None or buf.numel() < self._free[best].numel()):
                best = i
        if best is not None:
            return self._free.pop(best)
        size = 256
        while size < n:
            size *= 2
        return torch.empty(size, dtype=torch.int32).pin_memory()

    def release(self, buf: torch.Tensor) -> None:
        if len(self._free) < 32:
            self._free.append(buf)

    def upload(self, host: np.ndarray, device) -> torch.Tensor:
        """``host`` (int32) as a fresh device tensor; the copy is asynchronous on the current stream."""
        n = int(host.shape[0])
        buf = self.acquire(n)
        buf.numpy()[:n] = host
        dev = buf[:n].to(device, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._in_flight.append((buf, ev))
        return dev


_POOL = None


def pinned_pool() -> PinnedPool:
    global _POOL
    if _POOL is None:
        _POOL = PinnedPool()
    return _POOL
