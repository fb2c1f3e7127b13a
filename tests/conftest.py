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


def randn(shape, seed, std=1.0, dtype=torch.float32):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")
