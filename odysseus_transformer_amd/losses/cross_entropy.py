"""Fused softmax cross-entropy with in-place backward: the loss module the reference's training
loop takes from flash_attn (`from flash_attn.losses.cross_entropy import CrossEntropyLoss`,
train.py:8; built at train.py:173 with inplace_backward=True; applied at train.py:212-214 to
logits (T, V) and labels (T)), on the gfx950 HIP library."""
from __future__ import annotations

import torch
from torch import nn

from .. import _lib
from ..ops import _dt, _need_gpu, _stream


def _check(logits: torch.Tensor, labels: torch.Tensor) -> None:
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise ValueError(f"logits must be (tokens, vocab) with unit column stride, got {tuple(logits.shape)} "
                         f"stride {logits.stride()}")
    if labels.dtype != torch.int64 or tuple(labels.shape) != (logits.shape[0],) or labels.device != logits.device:
        raise ValueError(f"labels must be an int64 ({logits.shape[0]},) tensor on {logits.device}; got "
                         f"{labels.dtype} {tuple(labels.shape)} on {labels.device}")


def cross_entropy_fwd(logits, labels, ignore_index: int = -100):
    """-> losses (T) fp32, lse (T) fp32, reduced (2) fp32 = [mean over the counted tokens, their number]."""
    _need_gpu(logits, labels)
    _check(logits, labels)
    labels = labels.contiguous()
    T, V = logits.shape
    losses = torch.empty(T, dtype=torch.float32, device=logits.device)
    lse = torch.empty(T, dtype=torch.float32, device=logits.device)
    reduced = torch.empty(2, dtype=torch.float32, device=logits.device)
    _lib.call("ody_cross_entropy_fwd", logits.data_ptr(), labels.data_ptr(), losses.data_ptr(), lse.data_ptr(),
              reduced.data_ptr(), T, V, logits.stride(0), int(ignore_index), _dt(logits), _stream())
    return losses, lse, reduced


def cross_entropy_bwd_(logits, labels, lse, ignore_index: int = -100, reduced=None, grad_loss=None, dloss=None) -> None:
    """Overwrites `logits` with its gradient.  Either `dloss` (T) fp32, or `reduced` and the device
    scalar `grad_loss` for the mean reduction."""
    _need_gpu(logits, labels, lse, reduced, grad_loss, dloss)
    _check(logits, labels)
    T, V = logits.shape
    for t, n, numel in ((lse, "lse", T), (dloss, "dloss", T), (reduced, "reduced", 2), (grad_loss, "grad_loss", 1)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != numel or not t.is_contiguous()):
            raise ValueError(f"{n} must be a contiguous float32 tensor of {numel} elements, got {t.dtype} {tuple(t.shape)}")
    ptr = lambda t: 0 if t is None else t.data_ptr()
    _lib.call("ody_cross_entropy_bwd", logits.data_ptr(), labels.contiguous().data_ptr(), lse.data_ptr(), ptr(reduced),
              ptr(grad_loss), ptr(dloss), T, V, logits.stride(0), int(ignore_index), _dt(logits), _stream())


class CrossEntropyLossFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, ignore_index, reduction, inplace_backward):
        losses, lse, reduced = cross_entropy_fwd(logits, labels, ignore_index)
        ctx.save_for_backward(logits, labels, lse, reduced)
        ctx.ignore_index, ctx.reduction, ctx.inplace_backward = ignore_index, reduction, inplace_backward
        if reduction == "mean":
            return reduced[0]
        if reduction == "sum":
            return reduced[0] * reduced[1]
        return losses

    @staticmethod
    def backward(ctx, grad):
        logits, labels, lse, reduced = ctx.saved_tensors
        if not ctx.inplace_backward:
            logits = logits.clone()
        grad = grad.to(torch.float32)
        if ctx.reduction == "mean":
            cross_entropy_bwd_(logits, labels, lse, ctx.ignore_index, reduced=reduced,
                               grad_loss=grad.reshape(1).contiguous())
        else:
            dloss = grad.expand(logits.shape[0]).contiguous() if ctx.reduction == "sum" else grad.contiguous()
            cross_entropy_bwd_(logits, labels, lse, ctx.ignore_index, dloss=dloss)
        return logits, None, None, None, None


class CrossEntropyLoss(nn.Module):
    """Constructor keywords as flash_attn's module.  inplace_backward=True writes the gradient over
    the logits' own storage in backward (the logits are dead after the loss in a training step),
    saving one (tokens, vocab) allocation.  Label smoothing, the z-loss and vocabulary-parallel
    logits (process_group) are not implemented; the training loop uses none of them.

    Labels: `ignore_index` leaves a token out (loss 0, gradient row 0, not counted in the mean).  Any other
    label outside [0, vocab) gives that token the loss NaN, which every reduction then shows (its gradient row
    is 0: the kernels never index out of the row).  One deviation from flash_attn's module: the mean over ZERO
    counted tokens is 0 here, not the NaN of 0 / 0."""

    def __init__(self, ignore_index=-100, reduction="mean", label_smoothing=0.0, lse_square_scale=0.0,
                 inplace_backward=False, process_group=None):
        super().__init__()
        if reduction not in ("mean", "none", "sum"):
            raise NotImplementedError("Only support reduction = 'mean' or 'none' or 'sum'")
        if label_smoothing != 0.0 or lse_square_scale != 0.0 or process_group is not None:
            raise NotImplementedError("label_smoothing, lse_square_scale and process_group are not implemented")
        self.ignore_index = ignore_index
        self.reduction = reduction
        self.inplace_backward = inplace_backward

    def forward(self, input, target):
        assert input.is_cuda and target.is_cuda, "Only support CUDA tensors"
        return CrossEntropyLossFunction.apply(input, target, self.ignore_index, self.reduction, self.inplace_backward)
