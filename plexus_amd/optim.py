"""AdamW over flat fp32 tensors as one fused kernel per tensor.

Counterpart of ``torch.optim.AdamW(params, lr, weight_decay)`` as the reference's training script
builds it (examples/train.py:155-159): decoupled weight decay, default betas (0.9, 0.999), eps 1e-8, no
amsgrad.  The reference's optimizer runs a chain of elementwise kernels over every tensor; for the
trained input features (hundreds of millions of elements) that chain is a large share of an epoch, so
the update is done in one pass here.
"""
import torch

from . import _lib
from .ops import _need_gpu, _stream


class AdamW(torch.optim.Optimizer):
    """``shadows`` maps an fp32 master tensor to the bf16 tensor the model actually reads: the gradient is
    taken from the shadow (bf16), the update is applied to the master, and the shadow is refreshed in the
    same pass."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, shadows=None):
        if lr < 0 or eps < 0 or not (0 <= betas[0] < 1) or not (0 <= betas[1] < 1) or weight_decay < 0:
            raise ValueError("invalid AdamW hyper-parameters")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self.shadows = {id(m): (m, s) for m, s in (shadows or [])}

    def zero_grad(self, set_to_none=True):
        super().zero_grad(set_to_none)
        for _, s in self.shadows.values():
            if set_to_none:
                s.grad = None
            elif s.grad is not None:
                s.grad.zero_()

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        lib = _lib.load()
        for group in self.param_groups:
            b1, b2 = group["betas"]
            for p in group["params"]:
                shadow = self.shadows.get(id(p), (None, None))[1]
                grad = shadow.grad if shadow is not None else p.grad
                if grad is None:
                    continue
                _need_gpu(p, grad)
                if p.dtype != torch.float32 or not p.is_contiguous():
                    raise TypeError("plexus_amd.optim.AdamW updates contiguous fp32 tensors only")
                g = grad.contiguous()
                st = self.state[p]
                if not st:
                    st["step"] = 0
                    st["exp_avg"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                    st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                st["step"] += 1
                if g.dtype == torch.bfloat16:
                    if shadow is not None and (shadow.numel() != p.numel() or not shadow.is_contiguous()):
                        raise ValueError("bf16 shadow must be contiguous and as large as its master")
                    _lib.check(
                        lib.plx_adamw_f32_grad_bf16(p.numel(), p.data_ptr(), g.data_ptr(), st["exp_avg"].data_ptr(),
                                                    st["exp_avg_sq"].data_ptr(), group["lr"], b1, b2, group["eps"],
                                                    group["weight_decay"], st["step"],
                                                    shadow.data_ptr() if shadow is not None else None, _stream()),
                        "plx_adamw_f32_grad_bf16",
                    )
                else:
                    _lib.check(
                        lib.plx_adamw_f32(p.numel(), p.data_ptr(), g.data_ptr(), st["exp_avg"].data_ptr(),
                                          st["exp_avg_sq"].data_ptr(), group["lr"], b1, b2, group["eps"],
                                          group["weight_decay"], st["step"], _stream()),
                        "plx_adamw_f32",
                    )
        return loss
