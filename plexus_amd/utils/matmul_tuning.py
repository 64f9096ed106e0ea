"""Dense product entry of the layer; counterpart of plexus/utils/matmul_tuning.py:80-124.

The reference times eight transposition / layout variants of ``torch.mm`` per named product and keeps
the fastest; every variant computes ``A @ B``.  Here the product goes to the MFMA kernels, which read
both operands along contiguous memory whatever the transposition, so there is nothing to tune: the
name is accepted for interface compatibility and the transposed views the reference passes
(``torch.t(agg)``, ``torch.t(weight)``) are recognised and routed to the matching kernel.
"""
import torch

from .. import ops


def _is_transposed_view(t: torch.Tensor) -> bool:
    return t.dim() == 2 and t.stride(0) == 1 and t.shape[0] > 1 and t.stride(1) >= t.shape[0]


def tuned_matmul(A: torch.Tensor, B: torch.Tensor, matmul_name: str = "") -> torch.Tensor:
    """``A @ B`` on the matrix cores (fp32)."""
    if _is_transposed_view(A) and not _is_transposed_view(B):
        return ops.gemm_tn(A.t(), B)
    if _is_transposed_view(B) and not _is_transposed_view(A):
        return ops.gemm_nt(A, B.t())
    return ops.gemm_nn(A, B)
