"""Shared test plumbing: markers, import paths, tolerances, seeded inputs."""
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
for p in (ROOT, ROOT / "oracle"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

# Tolerances of the parity bar.  "Relative error" is the largest absolute
# difference divided by the largest magnitude of the oracle's tensor: an
# element-wise ratio is meaningless for entries that are zero by symmetry.
TOL_F32 = 1e-4     # fp32 kernels vs. fp32/fp64 oracle
TOL_BF16 = 2e-2    # bf16 kernels vs. fp32 oracle fed the same bf16-rounded inputs
TOL_LSE = 1e-3     # log-sum-exp, absolute and relative


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def rel_err(a: torch.Tensor, ref: torch.Tensor, floor: float = 1e-3) -> float:
    a, ref = a.detach().double().cpu(), ref.detach().double().cpu()
    # the floor keeps a tensor that is zero by construction (e.g. dq of a
    # single-key softmax) from turning rounding noise into a ratio of 1
    den = max(ref.abs().max().item(), floor)
    return (a - ref).abs().max().item() / den


def block_rel_err(a: torch.Tensor, ref: torch.Tensor, floor: float = 1e-3, floor_frac: float = 1e-3,
                  seq_dim=None, block: int = 64) -> float:
    """Largest BLOCK-WISE relative error: the tensor is cut along its sequence dimension into blocks
    of `block` consecutive positions (separately for every batch entry and head); for each block,
    max |a - ref| over the block divided by max |ref| over the same block.

    Under a causal mask the rows of out / dq / dk / dv shrink like 1 / sqrt(position), so a
    whole-tensor normalisation is set by the first rows and says little about the rest of a long
    sequence: a result whose second half is missing passes it.  This metric holds every block of
    64 rows to the tolerance on the block's own scale.  It is not taken row by row because single
    rows can be ill-conditioned: a query whose softmax sits on one key has dS = P (dP - delta) ~ 0
    by cancellation, and the bf16 rounding of `out` that every flash-attention backward inherits
    through delta = sum(dO * out) then is 10 % of that row (measured on an exact-arithmetic
    emulation with only `out` rounded).  A block of neighbouring rows is not.

    seq_dim: the dimension along which rows are neighbours (default: 1 for (B, L, H, D), 0 for
    (L, H, D) and for matrices).  The denominator is floored at `floor_frac` of the tensor's
    largest magnitude and at `floor` (the same absolute floor as rel_err)."""
    a, ref = a.detach().double().cpu(), ref.detach().double().cpu()
    if ref.numel() == 0:
        return 0.0
    if ref.dim() < 2:
        return rel_err(a, ref, floor)
    if seq_dim is None:
        seq_dim = 1 if ref.dim() == 4 else 0
    err = (a - ref).abs().amax(-1).movedim(seq_dim, -1)        # (..., L)
    mag = ref.abs().amax(-1).movedim(seq_dim, -1)
    L = err.shape[-1]
    pad = (-L) % block
    if pad:
        err = torch.nn.functional.pad(err, (0, pad))
        mag = torch.nn.functional.pad(mag, (0, pad))
    err = err.reshape(*err.shape[:-1], -1, block).amax(-1)
    mag = mag.reshape(*mag.shape[:-1], -1, block).amax(-1)
    den = mag.clamp_min(max(floor_frac * ref.abs().max().item(), floor))
    return (err / den).max().item()


def assert_parity(a: torch.Tensor, ref: torch.Tensor, tol: float, what: str = "", floor: float = 1e-3,
                  seq_dim=None, block: int = 64) -> None:
    """The parity bar: whole-tensor AND block-wise relative error within `tol`."""
    g, r = rel_err(a, ref, floor), block_rel_err(a, ref, floor, seq_dim=seq_dim, block=block)
    assert g <= tol, f"{what}: whole-tensor relative error {g:.3e} > {tol}"
    assert r <= tol, f"{what}: block-wise relative error {r:.3e} > {tol}"


def randn(shape, seed, std=1.0, dtype=torch.float32):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")
