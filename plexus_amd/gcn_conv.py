"""GCN layer: counterpart of plexus/gcn_conv.py at one rank, on hand-written gfx950 kernels.

Forward  (plexus/gcn_conv.py:137-219):  AGG = A.H ; OUT = AGG.W
Backward (plexus/gcn_conv.py:222-296):  GRAD_W = AGG^T.G ; GRAD_AGG = G.W^T ; GRAD_H = A^T.GRAD_AGG

Every collective of the reference is the identity at one rank and is not issued.  The aggregation is
always done first, as in the reference.  Optionally the ReLU that the reference's model applies after
the layer (examples/train.py:77-78) is fused: forward into the epilogue of the OUT product, backward as
a mask applied while GRAD_OUT is read.
"""
import math

import torch
from torch.nn import Parameter

from . import ops
from . import plexus as plx
from .utils.general import pad_dimension
from .utils.timers import get_timers


def chunk_bounds(num_rows, max_rows_per_chunk=1000000):
    """Row ranges of the blocked aggregation (plexus/gcn_conv.py:77-91)."""
    num_chunks = (num_rows + max_rows_per_chunk - 1) // max_rows_per_chunk
    rows_per_chunk = num_rows // num_chunks
    return [
        (i * rows_per_chunk, num_rows if i == num_chunks - 1 else (i + 1) * rows_per_chunk)
        for i in range(num_chunks)
    ]


class GCNConvFunction(torch.autograd.Function):
    """Forward and backward of one GCN layer.

    Takes the reference's twelve positional inputs (plexus/gcn_conv.py:137-151); the three process
    groups and the two gather flags are accepted and unused at one rank.  ``fuse_relu`` and the dropout
    triple are additions.  The storage type follows ``x``: fp32 (the reference's) or bf16 with fp32
    accumulation; the weight is always the fp32 parameter.
    """

    @staticmethod
    def forward(
        ctx,
        x,
        edge_index,
        edge_index_t,
        weight,
        local_features_shape,
        local_weight_shape,
        all_gather_group=None,
        aggregation_all_reduce_group=None,
        combination_all_reduce_group=None,
        gather_features=False,
        gather_weights=False,
        layer_num=0,
        fuse_relu=False,
        dropout_p=0.0,
        dropout_seed=0,
        dropout_offset=0,
        transform_first=False,
    ):
        if transform_first:
            return GCNConvFunction._forward_transform_first(
                ctx, x, edge_index, edge_index_t, weight, local_features_shape, local_weight_shape, layer_num, fuse_relu)
        timers = get_timers()
        timers.start("gcn conv fwd")
        A = ops.as_csr(edge_index)
        At = ops.as_csr(edge_index_t)
        bf16 = x.dtype == torch.bfloat16
        if dropout_p > 0.0 and not fuse_relu:
            raise ValueError("fused dropout follows the fused ReLU: it needs fuse_relu=True")

        # layer-0 features arrive flat (plexus/gcn_conv.py:176-180)
        H = x.detach().reshape(local_features_shape)

        timers.start("AGG = A * H")
        if plx.block_agg:
            # blocked aggregation (plexus/gcn_conv.py:184-185): same rows, one launch per chunk of <= 1 M rows
            AGG = ops.chunked_spmm(A, H)
        else:
            AGG = ops.spmm(A, H)
        timers.stop("AGG = A * H")

        W = weight.detach().reshape(local_weight_shape)
        timers.start("OUT = AGG * W")
        BITS = None
        if bf16:
            # a hidden layer's mask (ReLU and dropout) also as one bit per element where the kernel writes it: the two
            # backward products then read 1/16 of the mask's bytes
            want_bits = fuse_relu and ops.bf16_bits_supported(W.shape[1], W.shape[0])
            OUT = ops.gemm_nt_bf16(AGG, ops.cast_bf16(W, transpose=True), relu=fuse_relu, dropout_p=dropout_p,
                                   seed=dropout_seed, offset=dropout_offset, want_bits=want_bits)
            if want_bits:
                OUT, BITS = OUT
        elif fuse_relu:
            # the mask (ReLU, and dropout where it applies) also as one bit per element, written by the product itself:
            # GRAD_AGG reads it in place of OUT
            OUT, BITS = ops.gemm_nn(AGG, W, relu=True, want_bits=True, dropout_p=dropout_p, seed=dropout_seed, offset=dropout_offset)
        else:
            OUT = ops.gemm_nn(AGG, W)
        timers.stop("OUT = AGG * W")

        # the reference saves AGG, weight and the transposed adjacency (plexus/gcn_conv.py:194)
        ctx.save_for_backward(AGG, weight, OUT if fuse_relu else None, BITS if fuse_relu else None)
        ctx.adj_t = At
        ctx.local_weight_shape = tuple(local_weight_shape)
        ctx.x_shape = x.shape
        ctx.layer_num = layer_num
        ctx.fuse_relu = fuse_relu
        ctx.bf16 = bf16
        ctx.transform_first = False
        ctx.grad_scale = 1.0 / (1.0 - dropout_p) if dropout_p > 0.0 else 1.0
        timers.stop("gcn conv fwd")
        return OUT

    # ---- re-associated product:  A.(H.W)  instead of the reference's  (A.H).W ----
    # The two are the same matrix; when the layer narrows (out < in) the sparse product then gathers rows
    # of `out` instead of `in` elements, and the gather volume is what the layer costs.  Backward likewise:
    # T = A^T.G, GRAD_W = H^T.T, GRAD_H = T.W^T.  fp32 results differ from the reference order by rounding only.
    @staticmethod
    def _forward_transform_first(ctx, x, edge_index, edge_index_t, weight, local_features_shape, local_weight_shape,
                                 layer_num, fuse_relu):
        bf16 = x.dtype == torch.bfloat16
        if bf16 and fuse_relu:
            raise ValueError("transform-first association with bf16 storage is implemented for layers without a fused ReLU")
        timers = get_timers()
        timers.start("gcn conv fwd")
        A = ops.as_csr(edge_index)
        H = x.detach().reshape(local_features_shape)
        W = weight.detach().reshape(local_weight_shape)
        d_out = local_weight_shape[1]
        quantum = 8 if bf16 else 4  # rows of Z padded to 16 bytes so that the gather uses 128-bit loads
        d_pad = (d_out + quantum - 1) // quantum * quantum
        timers.start("OUT = AGG * W")
        # the padding columns are never written: the SpMM carries them through as columns of their own, and every
        # consumer reads the first d_out columns only
        Z = torch.empty((H.shape[0], d_pad), dtype=x.dtype, device=H.device)
        if bf16:
            ops.copy_rows(ops.gemm_nt_bf16(H, ops.cast_bf16(W, transpose=True)), Z[:, :d_out])
        else:
            ops.gemm_nn(H, W, out=Z[:, :d_out])
        timers.stop("OUT = AGG * W")
        timers.start("AGG = A * H")
        OUTp = ops.spmm(A, Z)
        timers.stop("AGG = A * H")
        OUT = OUTp[:, :d_out]
        if fuse_relu:
            ops.relu(OUT, inplace=True)
        ctx.save_for_backward(H, weight, OUT if fuse_relu else None)
        ctx.adj_t = ops.as_csr(edge_index_t)
        ctx.local_weight_shape = tuple(local_weight_shape)
        ctx.x_shape = x.shape
        ctx.layer_num = layer_num
        ctx.fuse_relu = fuse_relu
        ctx.bf16 = bf16
        ctx.transform_first = True
        ctx.grad_scale = 1.0
        timers.stop("gcn conv fwd")
        return OUT

    @staticmethod
    def _backward_transform_first(ctx, grad_output):
        timers = get_timers()
        timers.start("gcn conv bwd")
        H, weight, out = ctx.saved_tensors
        W = weight.detach().reshape(ctx.local_weight_shape)
        d_out = ctx.local_weight_shape[1]
        quantum = 8 if ctx.bf16 else 4
        d_pad = (d_out + quantum - 1) // quantum * quantum
        m = grad_output.shape[0]
        whole = ops._whole_padded_rows(grad_output) if d_pad != d_out else None
        if not ctx.fuse_relu and d_pad == d_out and grad_output.is_contiguous():
            Gp = grad_output
        elif not ctx.fuse_relu and whole is not None and whole.shape[1] == d_pad:
            Gp = whole  # the gradient already lies in rows of d_pad elements (the loss writes it in the layout of its logits)
        else:
            Gp = torch.empty((m, d_pad), dtype=grad_output.dtype, device=grad_output.device)
            if ctx.fuse_relu:
                ops.relu_bwd(grad_output, out, out=Gp[:, :d_out])
            else:
                ops.copy_rows(grad_output, Gp[:, :d_out])
        timers.start("GRAD_H = A.T * GRAD_AGG")
        T = ops.spmm(ctx.adj_t, Gp)[:, :d_out]
        timers.stop("GRAD_H = A.T * GRAD_AGG")
        grad_weight = None
        if ctx.needs_input_grad[3]:
            timers.start("GRAD_W = AGG.T * GRAD_OUT")
            grad_weight = (ops.gemm_tn_bf16(H, T) if ctx.bf16 else ops.gemm_tn(H, T)).reshape(weight.shape)
            timers.stop("GRAD_W = AGG.T * GRAD_OUT")
        grad_x = None
        if ctx.needs_input_grad[0]:
            timers.start("GRAD_AGG = GRAD_OUT * W.T")
            grad_x = (ops.gemm_nt_bf16(T, ops.cast_bf16(W)) if ctx.bf16 else ops.gemm_nt(T, W)).reshape(ctx.x_shape)
            timers.stop("GRAD_AGG = GRAD_OUT * W.T")
        timers.stop("gcn conv bwd")
        return (grad_x, None, None, grad_weight) + (None,) * 13

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.transform_first:
            return GCNConvFunction._backward_transform_first(ctx, grad_output)
        timers = get_timers()
        timers.start("gcn conv bwd")
        agg, weight, out, bits = ctx.saved_tensors
        W = weight.detach().reshape(ctx.local_weight_shape)
        mask = out if ctx.fuse_relu else None
        grad_output = grad_output.contiguous()

        grad_weight = None
        if ctx.needs_input_grad[3]:
            timers.start("GRAD_W = AGG.T * GRAD_OUT")
            if ctx.bf16:
                grad_weight = ops.gemm_tn_bf16(agg, grad_output, mask=mask, alpha=ctx.grad_scale, mask_bits=bits)
            else:
                grad_weight = ops.gemm_tn(agg, grad_output, mask=mask, alpha=ctx.grad_scale, mask_bits=bits)
            grad_weight = grad_weight.reshape(weight.shape)
            timers.stop("GRAD_W = AGG.T * GRAD_OUT")

        grad_x = None
        if ctx.needs_input_grad[0]:
            timers.start("GRAD_AGG = GRAD_OUT * W.T")
            if ctx.bf16:
                grad_agg = ops.gemm_nt_bf16(grad_output, ops.cast_bf16(W), mask=mask, alpha=ctx.grad_scale, mask_bits=bits)
            else:
                grad_agg = ops.gemm_nt(grad_output, W, mask=mask, mask_bits=bits, alpha=ctx.grad_scale)
            timers.stop("GRAD_AGG = GRAD_OUT * W.T")

            timers.start("GRAD_H = A.T * GRAD_AGG")
            grad_x = ops.spmm(ctx.adj_t, grad_agg)
            timers.stop("GRAD_H = A.T * GRAD_AGG")
            grad_x = grad_x.reshape(ctx.x_shape)  # flat again for layer 0 (plexus/gcn_conv.py:271)

        timers.stop("gcn conv bwd")
        return (grad_x, None, None, grad_weight) + (None,) * 13


class GCNConv(torch.nn.Module):
    """Drop-in for plexus.gcn_conv.GCNConv (plexus/gcn_conv.py:299-411) on one GPU.

    ``weight`` is a flat fp32 Parameter of ``in_channels * out_channels`` elements holding the
    row-major (in, out) matrix, as the reference stores it.  It is drawn with
    ``kaiming_uniform_(a=sqrt(5))`` on an (in, out) tensor (plexus/gcn_conv.py:332-333) -- on the host
    generator, so that a seed reproduces the same weights on any device -- or taken from ``weight``.

    Additions: ``association`` selects the order of the two products (see above; the default is the
    reference's); ``fuse_relu`` folds the model's ReLU into the layer; ``dropout`` (with ``fuse_relu``) drops
    activations after the ReLU in training mode with a counter-based generator keyed by ``dropout_seed``;
    every training forward uses a fresh offset (``layer_num + 64 * call count``), which is a host-side
    counter: a recorded HIP graph replays the mask it was recorded with.  The storage type follows the
    input tensor.
    """

    def __init__(self, in_channels, out_channels, layer_num, weight=None, fuse_relu=False, dropout=0.0, dropout_seed=0,
                 association="reference", device=None, **kwargs):
        super().__init__()
        self.layer_num = layer_num
        self.gather_features = layer_num == 0
        self.gather_weights = True
        # group sizes are all 1: padding is the identity (plexus/utils/general.py:20-23)
        self.in_channels = pad_dimension(in_channels, 1, 1)
        self.out_channels = pad_dimension(out_channels, 1)
        self.local_in_channels = self.in_channels
        self.local_out_channels = self.out_channels
        self.fuse_relu = fuse_relu
        self.dropout = float(dropout)
        self.dropout_seed = int(dropout_seed)
        # "reference": (A.H).W as plexus/gcn_conv.py:188,211 always does; "transform_first": A.(H.W);
        # "auto": transform first when that makes the gathered rows span fewer 128-byte lines (fp32 only)
        if association not in ("reference", "transform_first", "auto"):
            raise ValueError("association must be 'reference', 'transform_first' or 'auto'")
        # decided on fp32 row lengths; bf16 rows are half as long, which narrows the same layers
        lines = lambda d: (d * 4 + 127) // 128
        self.transform_first = association == "transform_first" or (
            association == "auto" and lines((out_channels + 3) // 4 * 4) < lines(in_channels))
        self.forward_calls = 0
        if device is None:
            device = "cuda" if torch.cuda.is_available() else "cpu"
        if weight is None:
            full_weight = torch.empty(in_channels, out_channels)
            torch.nn.init.kaiming_uniform_(full_weight, a=math.sqrt(5))
        else:
            full_weight = torch.as_tensor(weight, dtype=torch.float32).reshape(in_channels, out_channels)
        self.weight = Parameter(full_weight.reshape(-1).clone().to(device), requires_grad=True)

    def next_dropout_offset(self):
        """Offset the next training forward will use (the oracle regenerates the mask from it)."""
        return self.layer_num + 64 * self.forward_calls

    def forward(self, x, edge_index_shards):
        edge_index, edge_index_t = edge_index_shards[self.layer_num % len(edge_index_shards)]
        p = self.dropout if self.training else 0.0
        offset = self.next_dropout_offset()
        if p > 0.0:
            self.forward_calls += 1
        return GCNConvFunction.apply(
            x,
            edge_index,
            edge_index_t,
            self.weight,
            (edge_index.shape[1], self.local_in_channels),
            (self.local_in_channels, self.local_out_channels),
            None,
            None,
            None,
            self.gather_features,
            self.gather_weights,
            self.layer_num,
            self.fuse_relu,
            p,
            self.dropout_seed,
            offset,
            self.transform_first and p == 0.0 and (x.dtype == torch.float32 or not self.fuse_relu),
        )
