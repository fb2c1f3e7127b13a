"""Host-side slicing of the token / position / target ids for each sequence-parallel
mode (utils/apply_seq_parallel.py:4-144 of the reference).  Pure integer indexing."""
from __future__ import annotations

import torch

_KEYS = ("local_input_ids", "local_position_ids", "local_target_ids")


def extract_local_ulysses(value, rank, world_size, device, dim=1):
    """Contiguous block `rank` of `world_size` along the sequence axis."""
    n = value.shape[dim] // world_size
    return value[:, rank * n:(rank + 1) * n].to(device)


def extract_local_zigzag_ring(value, rank, world_size, device, dim=1):
    """Chunks `rank` and `2*world_size - 1 - rank` of 2*world_size, concatenated (balanced causal work)."""
    chunks = value.chunk(2 * world_size, dim=dim)
    return torch.cat([chunks[rank], chunks[2 * world_size - rank - 1]], dim=dim).to(device)


def _pack(ids, pos, tgt):
    return dict(zip(_KEYS, (ids, pos, tgt)))


def prepare_ulysses_attn_inputs(input_ids, position_ids, target_ids, rank, world_size, device):
    cut = lambda t: None if t is None else extract_local_ulysses(t, rank, world_size, device)
    return _pack(cut(input_ids), cut(position_ids), cut(target_ids))


def prepare_odysseus_attn_inputs(input_ids, position_ids, target_ids, rank, world_size, device):
    """Tokens and targets are sliced; the position ids stay FULL: attention runs over the
    whole gathered sequence on this rank's heads."""
    cut = lambda t: None if t is None else extract_local_ulysses(t, rank, world_size, device)
    return _pack(cut(input_ids), position_ids.to(device), cut(target_ids))


def prepare_tpsp_attn_inputs(input_ids, position_ids, target_ids, rank, world_size, device):
    return prepare_odysseus_attn_inputs(input_ids, position_ids, target_ids, rank, world_size, device)


def prepare_dp_attn_inputs(input_ids, position_ids, target_ids, rank, world_size, device):
    return _pack(input_ids.to(device), position_ids.to(device), target_ids.to(device))


def prepare_zigzag_ring_attn_inputs(input_ids, position_ids, target_ids, rank, world_size, device):
    cut = lambda t: None if t is None else extract_local_zigzag_ring(t, rank, world_size, device)
    return _pack(cut(input_ids), cut(position_ids), cut(target_ids))


_MODES = {
    "ulysses": prepare_ulysses_attn_inputs,
    "odysseus": prepare_odysseus_attn_inputs,
    "tpsp": prepare_tpsp_attn_inputs,
    "dp": prepare_dp_attn_inputs,
    "ring": prepare_zigzag_ring_attn_inputs,
}


def prepare_attn_inputs(parallel_mode, *args, **kwargs):
    try:
        fn = _MODES[parallel_mode]
    except KeyError:
        raise ValueError(f"Invalid parallel_mode: {parallel_mode}") from None
    return fn(*args, **kwargs)
