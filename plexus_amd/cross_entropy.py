"""Cross-entropy loss: counterpart of plexus/cross_entropy.py at one rank, as one fused kernel.

The reference runs about fifteen elementwise and row-reduction operators and saves the softmax and
an int64 one-hot matrix for backward (plexus/cross_entropy.py:35-101).  Here one pass over the logits
produces the loss and (softmax - onehot) / num_nodes; backward multiplies by the upstream scalar.
Unlike the reference (plexus/cross_entropy.py:40,75-76) the inputs are not modified.
"""
import torch

from . import ops
from .utils.timers import get_timers


class TensorParallelCrossEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target, num_layers, num_nodes, num_classes):
        timers = get_timers()
        timers.start("cross entropy fwd")
        loss, dlogits = ops.softmax_xent(
            logits.detach(), target, num_nodes, num_classes, want_grad=logits.requires_grad
        )
        ctx.save_for_backward(dlogits)
        timers.stop("cross entropy fwd")
        return loss.reshape(())

    @staticmethod
    def backward(ctx, grad_output):
        timers = get_timers()
        timers.start("cross entropy bwd")
        (dlogits,) = ctx.saved_tensors
        grad_input = ops.scale_by_scalar(dlogits, grad_output)  # plexus/cross_entropy.py:114
        timers.stop("cross entropy bwd")
        return grad_input, None, None, None, None


def parallel_cross_entropy(logits, target, groups, num_nodes, num_classes):
    """Same signature as plexus/cross_entropy.py:117-120 (``groups`` = number of layers, unused at one rank)."""
    return TensorParallelCrossEntropy.apply(logits, target, groups, num_nodes, num_classes)
