"""Sequence all-gather of a batch-1 activation (utils/allgather.py:4-10 of the reference)."""
from .linear_tpsp import allgather_along_first_dim_from_model_parallel_region


def allgather_bsz1(x):
    bsz, seqlen, h = x.shape
    assert bsz == 1, f"Batch size {bsz} must be 1 for allgather_bsz1"
    x = allgather_along_first_dim_from_model_parallel_region(x)
    return x.view(bsz, -1, h)
