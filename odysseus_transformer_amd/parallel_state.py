"""Model-parallel group registry (the three getters the reference takes from
fairscale.nn.model_parallel.initialize: decoder/odysseus.py:18,73-74,
utils/linear_tpsp.py:13-16, utils/linear_zero3.py:12-16).

This build computes one rank's share on one GPU.  The registry therefore holds a
world size, a rank and an optional torch.distributed group, and the sharded
modules size their parameters from it exactly as the reference does; the
collectives themselves are not part of this build and the call sites raise for
world_size > 1.
"""
from __future__ import annotations

_WORLD_SIZE = 1
_RANK = 0
_GROUP = None


def initialize_model_parallel(model_parallel_size: int = 1, rank: int = 0, group=None) -> None:
    """Declares the model-parallel layout used to size sharded parameters."""
    global _WORLD_SIZE, _RANK, _GROUP
    if model_parallel_size < 1 or not (0 <= rank < model_parallel_size):
        raise ValueError(f"bad model-parallel layout: size={model_parallel_size} rank={rank}")
    _WORLD_SIZE, _RANK, _GROUP = int(model_parallel_size), int(rank), group


def destroy_model_parallel() -> None:
    initialize_model_parallel(1, 0, None)


def get_model_parallel_world_size() -> int:
    return _WORLD_SIZE


def get_model_parallel_rank() -> int:
    return _RANK


def get_model_parallel_group():
    return _GROUP


def divide_and_check_no_remainder(numerator: int, denominator: int) -> int:
    if numerator % denominator != 0:
        raise AssertionError(f"{numerator} is not divisible by {denominator}")
    return numerator // denominator


def require_single_rank(what: str) -> None:
    """Guards every place where the reference issues a collective."""
    if _WORLD_SIZE != 1:
        raise NotImplementedError(
            f"{what}: the all-gather / reduce-scatter of the model-parallel group is outside this build, "
            f"which computes one rank's share from the already gathered activation (world_size={_WORLD_SIZE})")
