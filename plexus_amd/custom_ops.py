"""The layer and the loss as ``torch.library`` custom operators (``torch.ops.plexus_amd.*``).

``GCNConvFunction`` and ``TensorParallelCrossEntropy`` mirror the reference's two autograd functions
(plexus/gcn_conv.py:137-296, plexus/cross_entropy.py:19-114).  The operators here are the same computation in the
form the dispatcher knows: tensors and integers in, tensors out, a shape-only ("fake") implementation and a
registered backward each, so that a model built from them can be traced (``torch.compile``, ``torch.export``)
without a graph break.  They run the same entry points of libplexus_hip in the same order, so the results are
bit-identical to the autograd-function path.

A CSR matrix travels as its three arrays plus its shape; the prepared form (int32 indices, row plan) is looked up
in a small least-recently-used cache keyed by the arrays' addresses and built on first use; an entry holds the
arrays it was made from, so their addresses cannot pass to another matrix while it lives.

    out  = gcn_conv(x, A, At, weight, d_in, d_out, fuse_relu)      # A, At: ops.CsrMatrix or torch CSR tensors
    loss = cross_entropy(logits, target, num_nodes, num_classes)
"""
import collections
from typing import Tuple

import torch
from torch import Tensor

from . import ops


class _Entry:
    """A prepared matrix and the caller's arrays it was made from.  Holding the arrays keeps their memory from being
    freed and handed to another matrix while their addresses are the key; their version counters tell an in-place
    edit from an unchanged tensor."""

    __slots__ = ("rowptr", "col", "val", "versions", "csr")

    def __init__(self, rowptr, col, val, csr):
        self.rowptr, self.col, self.val, self.csr = rowptr, col, val, csr
        self.versions = (rowptr._version, col._version, val._version)


_PLANS = collections.OrderedDict()  # least recently used first
MAX_PLANS = 16  # a prepared matrix keeps its index arrays and its scratch (which can hold a copy of H) on the device


def clear_plan_cache() -> None:
    """Forget the prepared matrices (they keep their index arrays alive)."""
    _PLANS.clear()


def _remember(key, entry) -> None:
    _PLANS[key] = entry
    _PLANS.move_to_end(key)
    while len(_PLANS) > MAX_PLANS:
        _PLANS.popitem(last=False)


def _prepared(rowptr: Tensor, col: Tensor, val: Tensor, rows: int, cols: int) -> ops.CsrMatrix:
    key = (rowptr.data_ptr(), col.data_ptr(), val.data_ptr(), int(rows), int(cols), int(col.numel()))
    e = _PLANS.get(key)
    if e is not None and (e.rowptr._version, e.col._version) != e.versions[:2]:
        e = None  # the structure was edited in place: a new plan
    if e is None:
        e = _Entry(rowptr, col, val, ops.CsrMatrix(rowptr, col, val, (int(rows), int(cols))))
    elif e.val._version != e.versions[2]:
        if e.csr.val.data_ptr() != e.val.data_ptr():  # the prepared matrix holds a converted copy of the values: refresh it
            e.csr.val = e.val.to(torch.float32).contiguous()
        e.versions = e.versions[:2] + (e.val._version,)
    _remember(key, e)
    return e.csr


def _parts(a):
    """(rowptr, col, val, rows, cols) of a prepared matrix or a torch CSR tensor; a prepared matrix is entered
    into the cache under its own arrays, so it is not prepared twice."""
    a = ops.as_csr(a)
    key = (a.rowptr.data_ptr(), a.col.data_ptr(), a.val.data_ptr(), a.shape[0], a.shape[1], a.nnz)
    if key not in _PLANS:
        _remember(key, _Entry(a.rowptr, a.col, a.val, a))
    return a.rowptr, a.col, a.val, a.shape[0], a.shape[1]


# ---- AGG = A.H ; OUT = AGG.W (+ ReLU)          plexus/gcn_conv.py:184-212 ----
# The transposed matrix is an input of the forward operator although only the backward reads it: every tensor the
# backward needs is then visible to a tracer as an input or an output of the forward.  AGG is returned beside OUT for
# the same reason (the reference saves it, plexus/gcn_conv.py:194).
@torch.library.custom_op("plexus_amd::gcn_conv", mutates_args=())
def gcn_conv_op(x: Tensor, rowptr: Tensor, col: Tensor, val: Tensor, t_rowptr: Tensor, t_col: Tensor, t_val: Tensor, rows: int,
                cols: int, weight: Tensor, d_in: int, d_out: int, fuse_relu: bool) -> Tuple[Tensor, Tensor]:
    if x.dtype != torch.float32 or weight.dtype != torch.float32:
        raise TypeError("plexus_amd::gcn_conv takes fp32 features and weights")
    a = _prepared(rowptr, col, val, rows, cols)
    agg = ops.spmm(a, x.reshape(cols, d_in))
    out = ops.gemm_nn(agg, weight.reshape(d_in, d_out), relu=fuse_relu)
    return out, agg


@gcn_conv_op.register_fake
def _(x, rowptr, col, val, t_rowptr, t_col, t_val, rows, cols, weight, d_in, d_out, fuse_relu):
    return x.new_empty((rows, d_out)), x.new_empty((rows, d_in))


# ---- GRAD_W = AGG^T.G ; GRAD_AGG = G.W^T ; GRAD_H = A^T.GRAD_AGG          plexus/gcn_conv.py:236-266 ----
@torch.library.custom_op("plexus_amd::gcn_conv_bwd", mutates_args=())
def gcn_conv_bwd(grad_out: Tensor, agg: Tensor, out: Tensor, weight: Tensor, t_rowptr: Tensor, t_col: Tensor, t_val: Tensor,
                 rows: int, cols: int, d_in: int, d_out: int, fuse_relu: bool) -> Tuple[Tensor, Tensor]:
    at = _prepared(t_rowptr, t_col, t_val, cols, rows)
    mask = out if fuse_relu else None
    grad_out = grad_out.contiguous()
    w = weight.reshape(d_in, d_out)
    grad_w = ops.gemm_tn(agg, grad_out, mask=mask).reshape(weight.shape)
    grad_x = ops.spmm(at, ops.gemm_nt(grad_out, w, mask=mask))
    return grad_x, grad_w


@gcn_conv_bwd.register_fake
def _(grad_out, agg, out, weight, t_rowptr, t_col, t_val, rows, cols, d_in, d_out, fuse_relu):
    return grad_out.new_empty((cols, d_in)), torch.empty_like(weight)


def _conv_setup(ctx, inputs, output):
    x, rowptr, col, val, t_rowptr, t_col, t_val, rows, cols, weight, d_in, d_out, fuse_relu = inputs
    out, agg = output
    ctx.save_for_backward(agg, out, weight, t_rowptr, t_col, t_val)
    ctx.dims = (rows, cols, d_in, d_out, fuse_relu, x.shape)


def _conv_backward(ctx, grad_out, grad_agg):
    agg, out, weight, t_rowptr, t_col, t_val = ctx.saved_tensors
    rows, cols, d_in, d_out, fuse_relu, x_shape = ctx.dims
    grad_x, grad_w = gcn_conv_bwd(grad_out, agg, out, weight, t_rowptr, t_col, t_val, rows, cols, d_in, d_out, fuse_relu)
    return (grad_x.reshape(x_shape), None, None, None, None, None, None, None, None, grad_w, None, None, None)


gcn_conv_op.register_autograd(_conv_backward, setup_context=_conv_setup)


def gcn_conv(x: Tensor, a, at, weight: Tensor, d_in: int, d_out: int, fuse_relu: bool = False) -> Tensor:
    """One GCN layer, (A.H).W with an optional fused ReLU, through the dispatcher.  ``x`` may be flat (layer 0)."""
    rowptr, col, val, rows, cols = _parts(a)
    t_rowptr, t_col, t_val, t_rows, t_cols = _parts(at)
    if (t_rows, t_cols) != (cols, rows):
        raise ValueError("the second matrix must be the transpose of the first (%dx%d vs %dx%d)" % (t_rows, t_cols, rows, cols))
    out, _ = gcn_conv_op(x, rowptr, col, val, t_rowptr, t_col, t_val, rows, cols, weight, int(d_in), int(d_out), bool(fuse_relu))
    return out


# ---- masked row-softmax cross-entropy          plexus/cross_entropy.py:35-101, :111-114 ----
@torch.library.custom_op("plexus_amd::cross_entropy_fwd", mutates_args=())
def cross_entropy_fwd(logits: Tensor, target: Tensor, num_nodes: int, num_classes: int) -> Tuple[Tensor, Tensor]:
    loss, dlogits = ops.softmax_xent(logits, target, num_nodes, num_classes)
    return loss.reshape(()), dlogits


@cross_entropy_fwd.register_fake
def _(logits, target, num_nodes, num_classes):
    return logits.new_empty((), dtype=torch.float32), torch.empty_like(logits, memory_format=torch.contiguous_format)


@torch.library.custom_op("plexus_amd::scale_by_scalar", mutates_args=())
def scale_by_scalar(x: Tensor, scale: Tensor) -> Tensor:
    return ops.scale_by_scalar(x, scale)


@scale_by_scalar.register_fake
def _(x, scale):
    return torch.empty_like(x, memory_format=torch.contiguous_format)


def _xent_setup(ctx, inputs, output):
    ctx.save_for_backward(output[1])


def _xent_backward(ctx, grad_loss, grad_dlogits):
    (dlogits,) = ctx.saved_tensors
    return scale_by_scalar(dlogits, grad_loss), None, None, None


cross_entropy_fwd.register_autograd(_xent_backward, setup_context=_xent_setup)


def cross_entropy(logits: Tensor, target: Tensor, num_nodes: int, num_classes: int) -> Tensor:
    """Loss of plexus/cross_entropy.py:117-120 at one rank, through the dispatcher."""
    return cross_entropy_fwd(logits, target, int(num_nodes), int(num_classes))[0]
