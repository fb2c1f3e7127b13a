"""AdamW on the gfx950 HIP library: the optimizer of the reference's training loop
(torch.optim.AdamW(model.parameters(), lr=...), train.py:170,216) with the update of a tensor in ONE pass.

The host framework's default implementation runs the update as seven element-wise passes over every parameter
(about 1.2 TB/s of useful traffic on this chip); `ody_adamw` reads parameter, gradient and both moments once and
writes parameter and moments once.  Same hyper-parameters, same state layout (`step`, `exp_avg`, `exp_avg_sq`
per parameter, moments in the parameter's dtype), so state dicts interchange with torch.optim.AdamW; the
arithmetic is fp32 with one rounding per stored value, where the host rounds after each of its passes.
"""
from __future__ import annotations

import torch

from . import _lib


class AdamW(torch.optim.Optimizer):
    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8, weight_decay: float = 1e-2):
        if lr < 0.0 or eps < 0.0 or weight_decay < 0.0 or not 0.0 <= betas[0] < 1.0 or not 0.0 <= betas[1] < 1.0:
            raise ValueError(f"invalid hyper-parameters: lr={lr} betas={betas} eps={eps} weight_decay={weight_decay}")
        # the keys torch.optim.AdamW keeps in its parameter groups, so that a state dict saved here loads there with the
        # same meaning (a group without `decoupled_weight_decay` is read as plain Adam with L2 decay)
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=False, maximize=False,
                                      foreach=None, capturable=False, differentiable=False, fused=None,
                                      decoupled_weight_decay=True))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            b1, b2 = group["betas"]
            if group.get("amsgrad") or group.get("maximize") or group.get("decoupled_weight_decay", True) is False:
                raise NotImplementedError("amsgrad, maximize and coupled (L2) weight decay are not implemented")
            for p in group["params"]:
                if p.grad is None:
                    continue
                g = p.grad
                if g.is_sparse:
                    raise RuntimeError("AdamW does not support sparse gradients")
                if not p.is_cuda:
                    raise RuntimeError(f"odysseus_transformer_amd.optim.AdamW runs only on a HIP device (parameter is on "
                                       f"{p.device}); there is no CPU implementation in this package")
                if p.dtype not in (torch.bfloat16, torch.float32) or not p.is_contiguous():
                    raise ValueError(f"parameters must be contiguous bfloat16 or float32 tensors, got {p.dtype}")
                if g.dtype != p.dtype or not g.is_contiguous():
                    g = g.to(p.dtype).contiguous()
                state = self.state[p]
                if len(state) == 0:
                    state["step"] = torch.tensor(0.0)
                    state["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                state["step"] += 1
                _lib.call("ody_adamw", p.data_ptr(), g.data_ptr(), state["exp_avg"].data_ptr(),
                          state["exp_avg_sq"].data_ptr(), p.numel(), float(group["lr"]), float(b1), float(b2),
                          float(group["eps"]), float(group["weight_decay"]), int(state["step"].item()),
                          0 if p.dtype == torch.bfloat16 else 1, torch.cuda.current_stream(p.device).cuda_stream)
        return loss
