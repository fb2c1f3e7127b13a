"""`allgather_bsz1` (utils/allgather.py:4-10 of the reference): the sequence all-gather of a
(1, L/N, h) activation into (1, L, h).  The collective works on the leading dimension, so the
batch axis of extent 1 is what gets gathered and the result is re-viewed with it in front."""
from . import linear_tpsp as _tpsp


def allgather_bsz1(x):
    if x.dim() != 3 or x.shape[0] != 1:
        raise AssertionError(f"allgather_bsz1 takes a (1, seq, hidden) tensor, got {tuple(x.shape)}")
    hidden = x.shape[2]
    gathered = _tpsp.allgather_along_first_dim_from_model_parallel_region(x)
    return gathered.reshape(1, -1, hidden)
