"""Small arrays on their way to the device, and sampled tokens on their way back."""
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
        self.back = [None] * 4              # pinned buffers for the way back, used in turn
        self.back_turn = 0

    def upload(self, values: List, out: torch.Tensor = None, dtype: torch.dtype = torch.int32) -> torch.Tensor:
        """`values` (a list, or a tensor on the host) as an int32 or float32 tensor on the device
        (into `out`, if given: contiguous, with as many elements)."""
        data = values.to(dtype) if isinstance(values, torch.Tensor) else torch.tensor(values, dtype=dtype)
        if self.device.type != "cuda":
            if out is None:
                return data.clone() if data is values else data
            out.copy_(data.reshape(out.shape))
            return out
        index = self.turn
        self.turn = (index + 1) % len(self.buffers)
        if self.events[index] is not None:
            self.events[index].synchronize()
        count = data.numel()
        if self.buffers[index] is None or self.buffers[index].numel() < count:
            self.buffers[index] = torch.empty(max(count, 4096), dtype=torch.int32).pin_memory()
        host = self.buffers[index][:count].view(dtype)              # both types have four bytes
        host.copy_(data.reshape(-1))
        if out is None:
            out = torch.empty(count, dtype=dtype, device=self.device)
        out.view(-1).copy_(host, non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(self.device))
        self.events[index] = event
        return out


    def upload_filled(self, count: int, fill, out: torch.Tensor = None) -> torch.Tensor:
        """`count` int32 values that `fill(array)` writes into host memory (a numpy array of that length: pinned
        memory where the device is a GPU, so nothing is copied twice), as a tensor on the device (into `out`, if given)."""
        if self.device.type != "cuda":
            data = torch.empty(count, dtype=torch.int32)
            fill(data.numpy())
            if out is None:
                return data
            out.view(-1).copy_(data)
            return out
        index = self.turn
        self.turn = (index + 1) % len(self.buffers)
        if self.events[index] is not None:
            self.events[index].synchronize()
        if self.buffers[index] is None or self.buffers[index].numel() < count:
            self.buffers[index] = torch.empty(max(count, 4096), dtype=torch.int32).pin_memory()
        host = self.buffers[index][:count]
        fill(host.numpy())
        if out is None:
            out = torch.empty(count, dtype=torch.int32, device=self.device)
        out.view(-1).copy_(host, non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(self.device))
        self.events[index] = event
        return out

    def fetch(self, tensor: torch.Tensor) -> "Fetched":
        """Start copying a small int32 tensor to the host. Work queued on the device after this call does
        not delay the copy; at most as many fetches as there are buffers may be under way."""
        if self.device.type != "cuda":
            return Fetched(tensor.reshape(-1), None)
        index = self.back_turn
        self.back_turn = (index + 1) % len(self.back)
        count = tensor.numel()
        if self.back[index] is None or self.back[index].numel() < count:
            self.back[index] = torch.empty(max(count, 1024), dtype=torch.int32).pin_memory()
        host = self.back[index][:count]
        host.copy_(tensor.reshape(-1), non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(self.device))
        return Fetched(host, event)


class Fetched:
    """A few integers on their way from the device: `values()` waits for the copy, and only for it."""

    def __init__(self, host: torch.Tensor, event):
        self.host = host
        self.event = event

    def values(self) -> List[int]:
        if self.event is not None:
            self.event.synchronize()
        return self.host.tolist()


_STAGING = {}


def staging_for(device) -> Staging:
    device = torch.device(device)
    if device not in _STAGING:
        _STAGING[device] = Staging(device)
    return _STAGING[device]
