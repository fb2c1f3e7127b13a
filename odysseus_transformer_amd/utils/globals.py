"""Grow-only scratch arena keyed by (name, dtype) (utils/globals.py:9-41 of the
reference).  Callers must not use two tensors of the same key at the same time."""
from __future__ import annotations

import math

import torch

_GLOBAL_MEMORY_BUFFER = None


class GlobalMemoryBuffer:
    def __init__(self, dev):
        self.dev = dev
        self.buffer = {}

    def get_tensor(self, tensor_shape, dtype, name):
        """A view of `tensor_shape` on the arena slot (name, dtype); the slot grows, never shrinks."""
        need = math.prod(tensor_shape)
        slot = self.buffer.get((name, dtype))
        if slot is None or slot.numel() < need:
            slot = torch.empty(need, dtype=dtype, device=self.dev, requires_grad=False)
            self.buffer[(name, dtype)] = slot
        return slot[:need].view(*tensor_shape)


def _set_global_memory_buffer(dev):
    global _GLOBAL_MEMORY_BUFFER
    assert _GLOBAL_MEMORY_BUFFER is None, "global memory buffer is already initialized"
    _GLOBAL_MEMORY_BUFFER = GlobalMemoryBuffer(dev)


def _destroy_global_memory_buffer():
    global _GLOBAL_MEMORY_BUFFER
    _GLOBAL_MEMORY_BUFFER = None


def get_global_memory_buffer():
    assert _GLOBAL_MEMORY_BUFFER is not None, "global memory buffer is not initialized"
    return _GLOBAL_MEMORY_BUFFER
