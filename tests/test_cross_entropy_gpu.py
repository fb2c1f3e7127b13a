"""GPU parity of the fused cross-entropy (forward, in-place backward) against the oracle, which is
pinned to torch.nn.functional.cross_entropy and its autograd gradient in tests/test_oracle.py."""
import pytest
import torch

from conftest import TOL_BF16, TOL_F32, randn, rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu


def _labels(T, V, seed, ignore_every=0):
    y = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(seed))
    if ignore_every:
        y[::ignore_every] = -100
    return y


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("T,V,ignore_every", [(64, 32000, 0), (257, 32003, 7), (5, 7, 2), (1024, 128256, 0), (3, 50, 1)])
def test_cross_entropy_fwd_bwd(T, V, ignore_every, dtype, dev):
    from odysseus_transformer_amd.losses.cross_entropy import CrossEntropyLoss
    print(f"cross entropy T={T} V={V} ignore_every={ignore_every} {dtype}", flush=True)
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    x = randn((T, V), 11, std=2.0, dtype=dtype)
    y = _labels(T, V, 12, ignore_every)
    loss_ref, losses_ref, lse_ref, dx_ref = oracle.cross_entropy_fwd_bwd(x.float(), y, grad_loss=0.5)
    xg = x.to(dev).requires_grad_(True)
    logits = xg * 1.0                                 # a non-leaf, as the output of lm_head is
    keep = logits.detach().clone()
    loss = CrossEntropyLoss(inplace_backward=True)(logits, y.to(dev))
    assert loss.dtype == torch.float32 and loss.dim() == 0
    assert abs(loss.item() - loss_ref.item()) <= 1e-5 * max(1.0, abs(loss_ref.item()))
    (loss * 0.5).backward()
    assert rel_err(xg.grad, dx_ref) <= tol
    # the gradient was written over the logits' own storage
    assert torch.equal(logits.detach(), xg.grad) or ignore_every == 1
    # out of place: the logits survive
    xg2 = x.to(dev).requires_grad_(True)
    logits2 = xg2 * 1.0
    CrossEntropyLoss(inplace_backward=False)(logits2, y.to(dev)).backward(torch.tensor(0.5, device=dev))
    assert torch.equal(logits2.detach(), keep) and torch.equal(xg2.grad, xg.grad)


def test_cross_entropy_reductions_and_padded_rows(dev):
    from odysseus_transformer_amd.losses.cross_entropy import CrossEntropyLoss, cross_entropy_fwd
    T, V = 96, 1000
    full = randn((T, V + 24), 3, std=1.5)
    x = full[:, :V]                                  # row stride 1024, 1000 columns used
    y = _labels(T, V, 4, 5)
    _, losses_ref, lse_ref, _ = oracle.cross_entropy_fwd_bwd(x.double(), y)
    xg = full.to(dev)[:, :V]
    assert xg.stride(0) == V + 24
    losses, lse, reduced = cross_entropy_fwd(xg, y.to(dev))
    assert torch.allclose(losses.cpu().double(), losses_ref, atol=1e-5, rtol=1e-5)
    assert torch.allclose(lse.cpu().double(), lse_ref, atol=1e-5, rtol=1e-5)
    assert reduced[1].item() == (y != -100).sum().item()
    for red in ("none", "sum"):
        xr = xg.contiguous().requires_grad_(True)
        out = CrossEntropyLoss(reduction=red)(xr, y.to(dev))
        w = torch.linspace(0.5, 1.5, T, device=dev) if red == "none" else torch.tensor(2.0, device=dev)
        out.backward(w)
        xc = x.double().requires_grad_(True)
        ref = torch.nn.functional.cross_entropy(xc, y, reduction=red)
        ref.backward(w.cpu().double())
        assert torch.allclose(out.cpu().double(), ref.detach(), atol=1e-4, rtol=1e-5)
        assert rel_err(xr.grad, xc.grad) <= TOL_F32
    with pytest.raises(NotImplementedError):
        CrossEntropyLoss(label_smoothing=0.1)
    with pytest.raises(ValueError):
        cross_entropy_fwd(xg, y.to(dev).int())


def test_cross_entropy_training_shape(dev):
    """One training step's loss: 16384 tokens x 32000 vocabulary entries in bf16 (train.py:196-214)."""
    from odysseus_transformer_amd.losses.cross_entropy import CrossEntropyLoss
    T, V = 16384, 32000
    print("cross entropy 16384 x 32000 bf16", flush=True)
    x = randn((T, V), 21, std=1.0, dtype=torch.bfloat16)
    y = _labels(T, V, 22)
    loss_ref, _, _, dx_ref = oracle.cross_entropy_fwd_bwd(x.float(), y)
    logits = x.to(dev).requires_grad_(True) * 1.0
    loss = CrossEntropyLoss(inplace_backward=True)(logits, y.to(dev))
    loss.backward(loss)                              # the reference passes the loss itself as the gradient
    _, _, _, dx_ref = oracle.cross_entropy_fwd_bwd(x.float(), y, grad_loss=loss_ref.item())
    assert abs(loss.item() - loss_ref.item()) <= 1e-5 * loss_ref.item()
    assert rel_err(logits.detach(), dx_ref) <= TOL_BF16


def test_cross_entropy_label_out_of_range_is_loud(dev):
    """A label outside [0, V) that is not ignore_index makes the loss NaN (never a token silently dropped); the mean
    over zero counted tokens is 0 (the one documented deviation from 0 / 0)."""
    from odysseus_transformer_amd.losses.cross_entropy import CrossEntropyLoss, cross_entropy_fwd
    T, V = 16, 100
    x = randn((T, V), 21).to(dev)
    y = _labels(T, V, 22).to(dev)
    bad = y.clone()
    bad[3] = V          # off by one
    losses, _, reduced = cross_entropy_fwd(x, bad)
    assert torch.isnan(losses[3]) and not torch.isnan(losses[[0, 1, 2, 4]]).any()
    assert torch.isnan(reduced[0]) and reduced[1].item() == T
    xg = x.clone().requires_grad_(True)
    loss = CrossEntropyLoss(reduction="sum")(xg, bad)
    assert torch.isnan(loss)
    bad[3] = -5
    assert torch.isnan(CrossEntropyLoss()(x, bad))
    none = torch.full((T,), -100, dtype=torch.int64, device=dev)
    assert CrossEntropyLoss()(x, none).item() == 0.0
