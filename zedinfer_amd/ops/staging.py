"""Pinned host buffers for the small arrays a step copies to the device."""
from __future__ import annotations

from typing import List, Optional

import torch


class StagingRing:
    """A few pinned host buffers used in turn for the step's one copy to the device.  A buffer is
    written again only after the copy that last read it has finished."""

    def __init__(self, device: torch.device, depth: int = 4):
        self.device = device
        self.pinned = device.type == "cuda"
        self.buffers: List[Optional[torch.Tensor]] = [None] * depth
        self.events: List[Optional[torch.cuda.Event]] = [None] * depth
        self.turn = 0

    def acquire(self, n: int) -> torch.Tensor:
        self.turn = (self.turn + 1) % len(self.buffers)
        ev = self.events[self.turn]
        if ev is not None:
            ev.synchronize()
        buf = self.buffers[self.turn]
        if buf is None or buf.numel() < n:
            buf = torch.empty((max(n, 4096),), dtype=torch.int32, pin_memory=self.pinned)
            self.buffers[self.turn] = buf
        return buf[:n]

    def copied(self) -> None:
        """The copy out of the buffer last acquired has been queued on the current stream."""
        if self.pinned:
            ev = self.events[self.turn] or torch.cuda.Event()
            ev.record()
            self.events[self.turn] = ev
