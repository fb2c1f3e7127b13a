"""Process-wide scratch arena (same surface as utils/globals.py:9-41 of the reference).

One flat allocation per (name, dtype) key that only ever grows; `get_tensor` hands out a
view of its head.  Two tensors of one key alias each other: a caller holds at most one at a
time.  Sized for a 288 GB device: the largest users here are the attention backward's kept dS
(4 GiB at 4 heads x 32768 tokens) and the gathered (L, d) activation (256 MiB at L = 32768,
d = 4096).
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch


class GlobalMemoryBuffer:
    """name/dtype-keyed arena; `buffer` maps the key to its flat backing tensor."""

    def __init__(self, dev):
        self.dev = dev
        self.buffer: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}

    def get_tensor(self, tensor_shape, dtype, name):
        numel = 1
        for extent in tensor_shape:
            numel *= int(extent)
        key = (name, dtype)
        backing = self.buffer.get(key)
        if backing is None or backing.numel() < numel:   # first use, or a larger request: replace
            backing = self.buffer[key] = torch.empty(numel, dtype=dtype, device=self.dev, requires_grad=False)
        return backing.narrow(0, 0, numel).view(*tensor_shape)


class _Arena:
    """Holder of the singleton, so that the accessors below need no `global` statement."""
    instance: Optional[GlobalMemoryBuffer] = None


def _set_global_memory_buffer(dev):
    assert _Arena.instance is None, "global memory buffer is already initialized"
    _Arena.instance = GlobalMemoryBuffer(dev)


def _destroy_global_memory_buffer():
    _Arena.instance = None


def get_global_memory_buffer():
    assert _Arena.instance is not None, "global memory buffer is not initialized"
    return _Arena.instance
