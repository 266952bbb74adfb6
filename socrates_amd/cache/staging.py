"""Small host-to-device copies of integers (step inputs, block-table rows) through pinned
staging memory."""

from __future__ import annotations

import numpy as np
import torch


class PinnedUploader:
    """Host integers to the device without a pageable copy: a ring of pinned staging buffers,
    each followed by an event behind its last copy, so that the host never overwrites what a
    copy still reads and never waits in the usual case (the reference keeps persistent step
    buffers for the same reason, model/inference_paged.py:93-94, 185-188)."""

    def __init__(self, device, slots: int = 4, capacity: int = 1 << 14):
        self.device = torch.device(device)
        self._slots = [None] * slots
        self._events = [None] * slots
        self._capacity = capacity
        self._next = 0

    def __call__(self, array: np.ndarray, into: torch.Tensor = None) -> torch.Tensor:
        """int32 numpy array -> a device tensor of the same shape (a new one, or ``into``, a
        contiguous int32 device tensor of that many elements); the copy is queued on the
        current stream and reads a snapshot of ``array`` taken now."""
        n = int(array.size)
        out = into if into is not None else torch.empty(array.shape, dtype=torch.int32, device=self.device)
        if n == 0:
            return out
        i = self._next
        self._next = (i + 1) % len(self._slots)
        if self._events[i] is not None:
            self._events[i].synchronize()                 # the slot's last copy has read it
        buf = self._slots[i]
        if buf is None or buf.numel() < n:
            cap = max(self._capacity, 1 << (n - 1).bit_length())
            buf = self._slots[i] = torch.empty(cap, dtype=torch.int32).pin_memory()
        buf.numpy()[:n] = array.reshape(-1)
        out.view(-1).copy_(buf[:n], non_blocking=True)
        if self._events[i] is None:
            self._events[i] = torch.cuda.Event()
        self._events[i].record()
        return out


def pageable_upload(device):
    def upload(array: np.ndarray) -> torch.Tensor:
        return torch.from_numpy(np.ascontiguousarray(array, dtype=np.int32)).to(device)
    return upload
