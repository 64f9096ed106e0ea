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
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2):
        if lr < 0 or eps < 0 or not (0 <= betas[0] < 1) or not (0 <= betas[1] < 1) or weight_decay < 0:
            raise ValueError("invalid AdamW hyper-parameters")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))

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
                if p.grad is None:
                    continue
                _need_gpu(p, p.grad)
                if p.dtype != torch.float32 or not p.is_contiguous():
                    raise TypeError("plexus_amd.optim.AdamW updates contiguous fp32 tensors only")
                g = p.grad.contiguous()
                st = self.state[p]
                if not st:
                    st["step"] = 0
                    st["exp_avg"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                    st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                st["step"] += 1
                _lib.check(
                    lib.plx_adamw_f32(p.numel(), p.data_ptr(), g.data_ptr(), st["exp_avg"].data_ptr(),
                                      st["exp_avg_sq"].data_ptr(), group["lr"], b1, b2, group["eps"],
                                      group["weight_decay"], st["step"], _stream()),
                    "plx_adamw_f32",
                )
        return loss
