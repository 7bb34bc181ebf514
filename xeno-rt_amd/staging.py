"""Small integer arrays on their way to the device."""
from __future__ import annotations

from typing import List

import torch


class Staging:
    """Uploads small integer arrays to the device through a ring of pinned host buffers.

    The copy is asynchronous, so a host buffer must not be rewritten before the device has
    read it: each buffer carries an event that is waited for when its turn comes again
    (by then the copy has long been done, so the wait costs nothing).
    """

    def __init__(self, device, depth: int = 8):
        self.device = torch.device(device)
        self.buffers = [None] * depth
        self.events = [None] * depth
        self.turn = 0

    def upload(self, values: List[int], out: torch.Tensor = None) -> torch.Tensor:
        """`values` as an int32 tensor on the device (into `out`, if given)."""
        data = torch.tensor(values, dtype=torch.int32)
        if self.device.type != "cuda":
            if out is None:
                return data
            out.copy_(data)
            return out
        index = self.turn
        self.turn = (index + 1) % len(self.buffers)
        if self.events[index] is not None:
            self.events[index].synchronize()
        count = data.numel()
        if self.buffers[index] is None or self.buffers[index].numel() < count:
            self.buffers[index] = torch.empty(max(count, 4096), dtype=torch.int32).pin_memory()
        host = self.buffers[index][:count]
        host.copy_(data)
        if out is None:
            out = torch.empty(count, dtype=torch.int32, device=self.device)
        out.copy_(host, non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(self.device))
        self.events[index] = event
        return out


_STAGING = {}


def staging_for(device) -> Staging:
    device = torch.device(device)
    if device not in _STAGING:
        _STAGING[device] = Staging(device)
    return _STAGING[device]
