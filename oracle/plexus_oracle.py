"""CPU oracle for the Plexus GCN hot path.  TEST INFRASTRUCTURE ONLY.

This file restates, in stock CPU ``torch`` operators, what the reference computes on
its GCN hot path when every process group has one rank (all collectives are
identities, ``pad_dimension(d, 1) == d``).  It is the checker that the GPU kernels
are compared against; it is never imported by the product package.  Only tests,
the smoke check and the ``cpu_baseline`` leg of the benchmark may import it.

The arithmetic of the reference lives in a third-party dependency (PyTorch:
``torch.sparse.mm``, ``torch.mm`` and elementwise ops; unpinned in the
reference's requirements.txt:1).  The same operators are called here, at the
reference's own call sites and in the reference's order.  The reference holds
no tests, golden vectors or fixtures for this path, so every function below is
pinned by mathematics instead: dense matmul / scipy / brute-force loops for the
SpMM, numpy fp64 for the GEMMs, ``F.cross_entropy`` and autograd for the loss and
the backward formulas (see tests/test_oracle.py).

Every function takes ``dtype`` so that an fp64 twin of the same restatement can
arbitrate when two fp32 summation orders disagree.
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# plexus/utils/general.py
# --------------------------------------------------------------------------
def pad_dimension(dim_value: int, num_gpus: int, second_num_gpus: int = 1) -> int:
    """general.py:20-23 -- round ``dim_value`` up to a multiple of the group sizes."""
    prod = num_gpus * second_num_gpus
    rem = dim_value % prod
    return dim_value if rem == 0 else dim_value + prod - rem


# --------------------------------------------------------------------------
# CSR construction as the data loader does it (dataloader.py:343-368)
# --------------------------------------------------------------------------
def build_csr_pair(
    edge_index: torch.Tensor,
    edge_weight: torch.Tensor,
    shape: Tuple[int, int],
    row_range: Optional[Tuple[int, int]] = None,
    col_range: Optional[Tuple[int, int]] = None,
):
    """Mask edges to a block, re-base them, COO -> CSR and CSR of the transpose.

    Follows dataloader.py:343-368 (and benchmarking/spmm.py:67-84 for the block
    extraction): the transpose is materialised as its own CSR tensor.
    """
    if row_range is not None or col_range is not None:
        r0, r1 = row_range if row_range is not None else (0, shape[0])
        c0, c1 = col_range if col_range is not None else (0, shape[1])
        mask = (
            (edge_index[0] >= r0)
            & (edge_index[0] < r1)
            & (edge_index[1] >= c0)
            & (edge_index[1] < c1)
        )
        edge_index = edge_index[:, mask].clone()
        edge_index[0] -= r0
        edge_index[1] -= c0
        edge_weight = edge_weight[mask]
        shape = (r1 - r0, c1 - c0)
    coo = torch.sparse_coo_tensor(edge_index, edge_weight, shape)
    a = coo.to_sparse_csr()
    a_t = a.transpose(0, 1).to_sparse_csr()
    return a, a_t


# --------------------------------------------------------------------------
# GCN normalisation (consumed by the path; dataset.py:101, PyG T.GCNNorm)
# --------------------------------------------------------------------------
def gcn_norm(edge_index: torch.Tensor, num_nodes: int, edge_weight=None, dtype=torch.float32):
    """w_ij <- w_ij / sqrt(d_i d_j) after adding weight-1 self loops to nodes lacking one.

    PyG's GCNNorm is not in the reference tree (dataset.py:101 only calls it); its
    published definition is restated: existing self loops are kept, missing ones
    are filled with 1, the degree is the weighted in-degree by target index.
    """
    row, col = edge_index[0], edge_index[1]
    if edge_weight is None:
        edge_weight = torch.ones(row.numel(), dtype=dtype)
    edge_weight = edge_weight.to(dtype)
    has_loop = torch.zeros(num_nodes, dtype=torch.bool)
    has_loop[row[row == col]] = True
    missing = torch.nonzero(~has_loop).reshape(-1)
    row = torch.cat([row, missing])
    col = torch.cat([col, missing])
    w = torch.cat([edge_weight, torch.ones(missing.numel(), dtype=dtype)])
    deg = torch.zeros(num_nodes, dtype=dtype).index_add_(0, col, w)
    dinv = deg.pow(-0.5)
    dinv[torch.isinf(dinv)] = 0.0
    w = dinv[row] * w * dinv[col]
    return torch.stack([row, col]), w


def gcn_norm_csr_values(crow: torch.Tensor, col: torch.Tensor, val: torch.Tensor):
    """Symmetric normalisation applied to a CSR matrix that already holds its self loops.

    out_ij = val_ij / sqrt(d_i d_j) with d_i the sum of row i (for a symmetric
    matrix the row sum equals the column sum PyG uses).
    """
    m = crow.numel() - 1
    counts = crow[1:] - crow[:-1]
    rows = torch.repeat_interleave(torch.arange(m), counts)
    deg = torch.zeros(m, dtype=val.dtype).index_add_(0, rows, val)
    dinv = deg.pow(-0.5)
    dinv[torch.isinf(dinv)] = 0.0
    return dinv[rows] * val * dinv[col]


# --------------------------------------------------------------------------
# vertex permutation and 2-D partition files (plexus/utils/dataset.py, dataloader.py)
# --------------------------------------------------------------------------
def permute_graph(edge_index, edge_weight, x, y, perm, perm2=None, directed=False):
    """dataset.py:128-236 -- A = P.A.P2^T (and A2 = P2.A.P^T for the double permutation) through the same sparse
    products with permutation matrices P[i, perm[i]] = 1, then x = x[perm2], y = y[perm], y_2 = y[perm2].

    Returns a dict with the fields the reference stores on its data object.  Without ``perm2`` the single
    permutation of :189-193 (P2 = P) is applied.
    """
    n = x.shape[0]
    ar = torch.arange(n)
    ones = torch.ones(n, dtype=torch.float32)

    def pmat(p):
        return torch.sparse_coo_tensor(torch.stack([ar, p]), ones, (n, n)).to_sparse_csr()

    def to_edges(csr):  # to_edge_index: rows expanded from the row pointer, storage order
        crow = csr.crow_indices()
        rows = torch.repeat_interleave(torch.arange(n), crow[1:] - crow[:-1])
        return torch.stack([rows, csr.col_indices()]), csr.values()

    adj = torch.sparse_coo_tensor(edge_index, edge_weight, (n, n)).to_sparse_csr()
    if directed:
        adj = adj.transpose(0, 1).to_sparse_csr()
    P = pmat(perm)
    out = {}
    if perm2 is not None:
        P2 = pmat(perm2)
        a1 = torch.sparse.mm(torch.sparse.mm(P, adj), P2.transpose(0, 1).to_sparse_csr())
        a2 = torch.sparse.mm(torch.sparse.mm(P2, adj), P.transpose(0, 1).to_sparse_csr())
        out["edge_index"], out["edge_weight"] = to_edges(a1)
        out["edge_index_2"], out["edge_weight_2"] = to_edges(a2)
        out["x"] = x[perm2, :]
        out["y"] = y[perm]
        out["y_2"] = y[perm2]
    else:
        a1 = torch.sparse.mm(torch.sparse.mm(P, adj), P.transpose(0, 1).to_sparse_csr())
        out["edge_index"], out["edge_weight"] = to_edges(a1)
        out["x"] = x[perm, :]
        out["y"] = y[perm]
    return out


def load_partitioned(data_dir: str, num_gcn_layers: int, num_gpus=(1, 1, 1), ranks=(0, 0, 0)):
    """dataloader.py:47-151 (index ranges), :153-325 (merging partition files), :327-452 (cutting, padding),
    :454-540 (load) for a partitioned directory, on the host with stock torch operators.

    ``num_gpus`` and ``ranks`` are in the reference's ("z", "x", "y") order (:57).  Returns
    (adj_shards as torch CSR pairs, flat features, labels, num_nodes, num_features, num_classes).
    Vertex ids stay int64 when files are merged (the reference concatenates onto an empty fp32 tensor, :163,205,
    which would turn them into floats).
    """
    import glob
    import os

    double_perm = os.path.exists(os.path.join(data_dir, "edge_index", "1"))
    parts = len(glob.glob(os.path.join(data_dir, "output_labels", "0", "*.pt")))
    num_nodes, num_features, num_classes = torch.load(os.path.join(data_dir, "metadata.pt"), weights_only=True)

    nodes_step = pad_dimension(num_nodes, num_gpus[1]) // num_gpus[1]
    feats_step = pad_dimension(num_features, num_gpus[2], num_gpus[0]) // num_gpus[2]
    nodes_start, nodes_stop = ranks[1] * nodes_step, (ranks[1] + 1) * nodes_step
    feats_start, feats_stop = ranks[2] * feats_step, (ranks[2] + 1) * feats_step
    depth_step = pad_dimension((nodes_stop - nodes_start) * (feats_stop - feats_start), num_gpus[0]) // num_gpus[0]
    depth_start, depth_stop = ranks[0] * depth_step, (ranks[0] + 1) * depth_step
    if num_gcn_layers % 3 == 1:
        lg = 0
    elif num_gcn_layers % 3 == 2:
        lg = 2
    else:
        lg = 1
    labels_step = pad_dimension(num_nodes, num_gpus[lg]) // num_gpus[lg]
    labels_start, labels_stop = ranks[lg] * labels_step, (ranks[lg] + 1) * labels_step

    blocks = []
    for i in range(min(3, num_gcn_layers)):
        d1, d2 = ((0, 1), (2, 0), (1, 2))[i]
        s1 = pad_dimension(num_nodes, num_gpus[d1]) // num_gpus[d1]
        s2 = pad_dimension(num_nodes, num_gpus[d2]) // num_gpus[d2]
        blocks.append(((ranks[d1] * s1, (ranks[d1] + 1) * s1), (ranks[d2] * s2, (ranks[d2] + 1) * s2)))

    psize = pad_dimension(num_nodes, parts) // parts
    fsize = pad_dimension(num_features, parts) // parts

    def covering(start, stop, size):
        return range(min(start // size, parts), min(((stop - 1) // size) + 1, parts))

    adj_shards = []
    for layer in range(min(6 if double_perm else 3, num_gcn_layers)):
        (r0, r1), (c0, c1) = blocks[layer % 3]
        which = 1 if (double_perm and layer % 2 != 0) else 0
        idx = torch.empty((2, 0), dtype=torch.int64)
        val = torch.empty(0)
        for i in covering(r0, r1, psize):
            for j in covering(c0, c1, psize):
                ei, w = torch.load(os.path.join(data_dir, "edge_index", str(which), "%d_%d.pt" % (i, j)), weights_only=True)
                idx = torch.cat((idx, ei), dim=1)
                val = torch.cat((val, w), dim=0)
        adj_shards.append(build_csr_pair(idx, val, (num_nodes, num_nodes), (r0, r1), (c0, c1)))

    merged = None
    for i in covering(nodes_start, nodes_stop, psize):
        row = None
        for j in covering(feats_start, feats_stop, fsize):
            t = torch.load(os.path.join(data_dir, "input_features", "%d_%d.pt" % (i, j)), weights_only=True)
            row = t if row is None else torch.cat((row, t), dim=1)
        merged = row if merged is None else torch.cat((merged, row), dim=0)
    pn0 = (nodes_start // psize) * psize
    pf0 = (feats_start // fsize) * fsize
    if merged is None:
        merged = torch.zeros(nodes_stop - nodes_start, feats_stop - feats_start)
        pn0, pf0 = nodes_start, feats_start
    local = merged[nodes_start - pn0 : nodes_stop - pn0, feats_start - pf0 : feats_stop - pf0]
    local = F.pad(local, (0, (feats_stop - feats_start) - local.shape[1], 0, (nodes_stop - nodes_start) - local.shape[0]))
    features = local.reshape(-1)[depth_start:depth_stop]

    which = 1 if (double_perm and num_gcn_layers % 2 == 0) else 0
    labels = torch.empty(0, dtype=torch.int64)
    for i in covering(labels_start, labels_stop, psize):
        labels = torch.cat((labels, torch.load(os.path.join(data_dir, "output_labels", str(which), "%d.pt" % i), weights_only=True)))
    pl0 = (labels_start // psize) * psize
    labels = labels[labels_start - pl0 : labels_stop - pl0]
    labels = F.pad(labels, (0, (labels_stop - labels_start) - labels.shape[0])).to(torch.int64)
    return adj_shards, features, labels, num_nodes, num_features, num_classes


# --------------------------------------------------------------------------
# plexus/gcn_conv.py
# --------------------------------------------------------------------------
def extract_csr_submatrix(csr: torch.Tensor, start_row: int, end_row: int) -> torch.Tensor:
    """gcn_conv.py:25-64 -- rows [start_row, end_row) of a CSR matrix as a new CSR matrix."""
    crow = csr.crow_indices()
    col = csr.col_indices()
    val = csr.values()
    p0 = int(crow[start_row])
    p1 = int(crow[end_row])
    sub_crow = crow[start_row : end_row + 1] - p0
    return torch.sparse_csr_tensor(
        sub_crow, col[p0:p1], val[p0:p1], size=(end_row - start_row, csr.size(1)), dtype=csr.dtype
    )


def chunk_bounds(num_rows: int, max_rows_per_chunk: int = 1000000) -> List[Tuple[int, int]]:
    """gcn_conv.py:77-91 -- the row ranges of the blocked aggregation."""
    num_chunks = (num_rows + max_rows_per_chunk - 1) // max_rows_per_chunk
    rows_per_chunk = num_rows // num_chunks
    out = []
    for i in range(num_chunks):
        s = i * rows_per_chunk
        e = num_rows if i == num_chunks - 1 else (i + 1) * rows_per_chunk
        out.append((s, e))
    return out


def spmm(a_csr: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
    """gcn_conv.py:188 (forward) and :265 (backward, on the transposed CSR)."""
    return torch.sparse.mm(a_csr, h)


def chunked_spmm(a_csr: torch.Tensor, h: torch.Tensor, max_rows_per_chunk: int = 1000000) -> torch.Tensor:
    """gcn_conv.py:67-128 with a one-rank all-reduce group: SpMM per row chunk, concatenated."""
    parts = [
        torch.sparse.mm(extract_csr_submatrix(a_csr, s, e), h)
        for s, e in chunk_bounds(a_csr.size(0), max_rows_per_chunk)
    ]
    return torch.cat(parts, dim=0)


def gcn_conv_forward(x, a_csr, weight, local_features_shape, local_weight_shape, block_agg=False):
    """gcn_conv.py:137-219 at one rank.  Returns (OUT, AGG); AGG is what the reference saves."""
    h = x.reshape(local_features_shape)  # :176-180 (layer-0 input arrives flat)
    agg = chunked_spmm(a_csr, h) if block_agg else spmm(a_csr, h)  # :184-191
    w = weight.reshape(local_weight_shape)  # :207
    out = torch.mm(agg, w)  # :211 -> matmul_tuning.py:95
    return out, agg


def gcn_conv_backward(grad_output, agg, weight, a_t_csr, local_weight_shape, flatten_grad_x=False):
    """gcn_conv.py:222-296 at one rank.  Returns (grad_x, grad_weight_flat)."""
    w = weight.reshape(local_weight_shape)  # :232
    grad_weight = torch.mm(torch.t(agg), grad_output).reshape(-1)  # :237-239, :252
    grad_agg = torch.mm(grad_output, torch.t(w))  # :256-258
    grad_x = torch.sparse.mm(a_t_csr, grad_agg)  # :265
    if flatten_grad_x:  # :271 (layer 0)
        grad_x = grad_x.reshape(-1)
    return grad_x, grad_weight


def kaiming_uniform_weight(in_channels: int, out_channels: int, generator: torch.Generator, dtype=torch.float32):
    """gcn_conv.py:332-333 -- kaiming_uniform_(a=sqrt(5)) on an (in, out) tensor.

    torch computes fan_in from size(1), so fan_in = out_channels here; the bound is
    gain * sqrt(3 / fan_in) with gain = sqrt(2 / (1 + 5)) = 1 / sqrt(fan_in).  The values
    are drawn on a host generator so both paths share them.  Returned flat, as the
    reference stores the parameter (:372-390 at one rank).
    """
    bound = 1.0 / math.sqrt(out_channels)
    w = (torch.rand(in_channels, out_channels, generator=generator, dtype=torch.float64) * 2 - 1) * bound
    return w.to(dtype).reshape(-1)


# --------------------------------------------------------------------------
# plexus/cross_entropy.py
# --------------------------------------------------------------------------
def cross_entropy_forward(logits, target, num_nodes: int, num_classes: int):
    """cross_entropy.py:19-105 at one rank.  Inputs are not mutated (the reference mutates both).

    Returns (loss, softmax, onehot) -- the last two are what the reference saves.
    """
    logits = logits.clone()
    target = target.clone()
    m, c = logits.shape
    invalid_classes = torch.arange(c) >= num_classes  # :35-38
    logits[:, invalid_classes] = float("-inf")  # :40
    logits_max = torch.max(logits, dim=1)[0]  # :43
    numerator = torch.exp(logits - logits_max.unsqueeze(1))  # :49
    denominator = torch.sum(numerator, dim=1)  # :53
    softmax = numerator / denominator.unsqueeze(1)  # :57
    invalid_nodes = (torch.arange(m) >= num_nodes) | (target < 0)  # :60-66
    softmax[invalid_nodes, :] = 0.0  # :67
    invalid_logits_mask = (target < 0) | (target >= c)  # :70-72
    target[invalid_logits_mask] = 0  # :75-76
    onehot = F.one_hot(target, num_classes=c)  # :79
    onehot[invalid_logits_mask] = 0  # :82
    eps = 1e-9
    loss = torch.sum(-torch.log(softmax.clamp(min=eps)) * onehot, dim=1)  # :88-89
    loss_sum = torch.sum(loss)  # :97
    return loss_sum / num_nodes, softmax, onehot  # :101


def cross_entropy_backward(softmax, onehot, num_nodes: int, grad_output=1.0):
    """cross_entropy.py:108-114."""
    return (softmax - onehot) / num_nodes * grad_output


# --------------------------------------------------------------------------
# examples/train.py: Net + train()
# --------------------------------------------------------------------------
class OracleNet:
    """examples/train.py:55-79 with hand-written backward (gcn_conv.py:222-296).

    Layers are (A.H).W with ReLU after every layer except the last, no bias.  The weights
    (flat, as the reference keeps them) and the input features are the trained tensors.
    """

    def __init__(self, weights: Sequence[torch.Tensor], dims: Sequence[int], dropout_p: float = 0.0, seed: int = 0):
        self.weights = [w.clone() for w in weights]
        self.dims = list(dims)
        # dropout after every ReLU (not in the reference's Net; the counter-based mask of dropout_keep_mask below)
        self.p = dropout_p
        self.seed = seed

    def forward(self, x, adj_shards, offsets=None):
        """``offsets[i]``: dropout offset of layer i for this pass (needed when dropout_p > 0)."""
        saved = []
        h = x
        n_layers = len(self.weights)
        for i, w in enumerate(self.weights):
            a, a_t = adj_shards[i % len(adj_shards)]  # gcn_conv.py:394-396
            fshape = (a.shape[1], self.dims[i])
            wshape = (self.dims[i], self.dims[i + 1])
            out, agg = gcn_conv_forward(h, a, w, fshape, wshape)
            pre = out
            keep = None
            if i != n_layers - 1:
                out = F.relu(out)  # train.py:77-78
                if self.p > 0.0:
                    keep = torch.from_numpy(dropout_keep_mask(out.numel(), self.seed, offsets[i], self.p).reshape(out.shape)).to(out.dtype)
                    out = out * keep / (1.0 - self.p)
            saved.append((agg, a_t, wshape, pre, keep))
            h = out
        self._saved = saved
        return h

    def backward(self, grad_logits, masks=None):
        """``masks[i]`` (optional) replaces the ReLU mask ``pre_i > 0`` of layer i: a pre-activation within
        rounding of zero may take either sign in two fp32 summation orders, and a caller comparing backward
        passes can pin the mask to the one the other implementation used."""
        g = grad_logits
        grads_w = [None] * len(self.weights)
        n_layers = len(self.weights)
        for i in reversed(range(n_layers)):
            agg, a_t, wshape, pre, keep = self._saved[i]
            if i != n_layers - 1:
                mask = (pre > 0) if masks is None or masks[i] is None else masks[i]
                g = g * mask.to(g.dtype)
                if keep is not None:
                    g = g * keep / (1.0 - self.p)
            g, grads_w[i] = gcn_conv_backward(g, agg, self.weights[i], a_t, wshape, flatten_grad_x=(i == 0))
        return g, grads_w


def adamw_step(params, grads, state, lr=3e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0):
    """torch.optim.AdamW as examples/train.py:155-159 configures it (published update rule)."""
    state["t"] = state.get("t", 0) + 1
    t = state["t"]
    b1, b2 = betas
    for k, (p, g) in enumerate(zip(params, grads)):
        m = state.setdefault(("m", k), torch.zeros_like(p))
        v = state.setdefault(("v", k), torch.zeros_like(p))
        p.mul_(1 - lr * weight_decay)
        m.mul_(b1).add_(g, alpha=1 - b1)
        v.mul_(b2).addcmul_(g, g, value=1 - b2)
        denom = (v.sqrt() / math.sqrt(1 - b2**t)).add_(eps)
        p.addcdiv_(m, denom, value=-lr / (1 - b1**t))


def train_epochs(x0, weights, dims, adj_shards, labels, num_nodes, num_classes, epochs=10, lr=3e-3, masks_of_epoch=None):
    """examples/train.py:83-112,164-193: zero_grad -> fwd -> CE -> bwd -> AdamW over weights and features.

    Returns the loss of every epoch and the final (features, weights).  ``masks_of_epoch(e)`` (optional) gives the
    ReLU masks the backward pass of epoch e uses in place of its own (see OracleNet.backward).
    """
    net = OracleNet(weights, dims)
    x = x0.clone().reshape(-1)
    state = {}
    losses = []
    for e in range(epochs):
        logits = net.forward(x, adj_shards)
        loss, softmax, onehot = cross_entropy_forward(logits, labels, num_nodes, num_classes)
        g = cross_entropy_backward(softmax, onehot.to(softmax.dtype), num_nodes)
        gx, gws = net.backward(g, None if masks_of_epoch is None else masks_of_epoch(e))
        adamw_step(net.weights + [x], gws + [gx], state, lr=lr)
        losses.append(float(loss))
    return losses, x, net.weights


# --------------------------------------------------------------------------
# dropout (not in the reference; counter-based so host and device agree bit for bit)
# --------------------------------------------------------------------------
_PHILOX_M0 = np.uint64(0xD2511F53)
_PHILOX_M1 = np.uint64(0xCD9E8D57)
_PHILOX_W0 = np.uint32(0x9E3779B9)
_PHILOX_W1 = np.uint32(0xBB67AE85)


def philox4x32_10(counter: np.ndarray, key: Tuple[int, int]) -> np.ndarray:
    """Philox-4x32-10 (Salmon et al., SC'11) on an array of 4x uint32 counters, shape (n, 4)."""
    c = counter.astype(np.uint32).copy()
    k0 = np.uint32(key[0])
    k1 = np.uint32(key[1])
    mask = np.uint64(0xFFFFFFFF)
    with np.errstate(over="ignore"):
        for _ in range(10):
            p0 = _PHILOX_M0 * c[:, 0].astype(np.uint64)
            p1 = _PHILOX_M1 * c[:, 2].astype(np.uint64)
            hi0 = (p0 >> np.uint64(32)).astype(np.uint32)
            lo0 = (p0 & mask).astype(np.uint32)
            hi1 = (p1 >> np.uint64(32)).astype(np.uint32)
            lo1 = (p1 & mask).astype(np.uint32)
            n0 = hi1 ^ c[:, 1] ^ k0
            n2 = hi0 ^ c[:, 3] ^ k1
            c = np.stack([n0, lo1, n2, lo0], axis=1)
            k0 = np.uint32(k0 + _PHILOX_W0)
            k1 = np.uint32(k1 + _PHILOX_W1)
    return c


def dropout_keep_mask(n_elems: int, seed: int, offset: int, p: float) -> np.ndarray:
    """Keep-mask of the fused dropout (not in the reference; counter-based so host and device agree).

    Element e (row-major linear index) uses call q = e // 8 of Philox-4x32-10 with counter
    (q, offset) and key seed; its 16-bit lane is the low (e even) or high (e odd) half of output word
    (e % 8) // 2; the element is kept iff lane >= round(p * 65536).
    """
    n8 = (n_elems + 7) // 8
    ctr = np.zeros((n8, 4), dtype=np.uint32)
    idx = np.arange(n8, dtype=np.uint64)
    ctr[:, 0] = (idx & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    ctr[:, 1] = (idx >> np.uint64(32)).astype(np.uint32)
    ctr[:, 2] = np.uint32(offset & 0xFFFFFFFF)
    ctr[:, 3] = np.uint32((offset >> 32) & 0xFFFFFFFF)
    words = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))  # (n8, 4)
    lanes = np.empty((n8, 8), dtype=np.uint32)
    lanes[:, 0::2] = words & np.uint32(0xFFFF)
    lanes[:, 1::2] = words >> np.uint32(16)
    thresh = min(int(round(p * 65536.0)), 65535)
    return lanes.reshape(-1)[:n_elems] >= np.uint32(thresh)


# --------------------------------------------------------------------------
# bf16 storage with fp32 accumulation (not in the reference): the fp32 operator sequence above with
# every STORED tensor rounded to bf16, which is what the device path keeps in memory
# --------------------------------------------------------------------------
def rb(t: torch.Tensor) -> torch.Tensor:
    """Round to bf16 and back (round-to-nearest-even), keeping the working dtype."""
    return t.to(torch.bfloat16).to(t.dtype)


class OracleNetBf16:
    """OracleNet with bf16-stored activations, optional dropout after each ReLU, fp32 weights.

    forward:  AGG = rb(A.H); OUT = rb(dropout(relu(AGG . rb(W))))          (last layer: no ReLU / dropout)
    backward: G' = G * [OUT > 0] / (1 - p); GRAD_W = AGG^T . G' (fp32, not rounded);
              GRAD_AGG = rb(G' . rb(W)^T); GRAD_H = rb(A^T . GRAD_AGG)
    ``offsets[i]`` is the dropout offset of layer i for this forward pass.
    """

    def __init__(self, weights, dims, dropout_p=0.0, seed=0):
        self.weights = [w.clone() for w in weights]
        self.dims = list(dims)
        self.p = dropout_p
        self.seed = seed

    def forward(self, x, adj_shards, offsets=None):
        saved = []
        h = rb(x)
        n_layers = len(self.weights)
        for i, w in enumerate(self.weights):
            a, a_t = adj_shards[i % len(adj_shards)]
            agg = rb(torch.sparse.mm(a, h.reshape(a.shape[1], self.dims[i])))
            out = torch.mm(agg, rb(w.reshape(self.dims[i], self.dims[i + 1])))
            last = i == n_layers - 1
            if not last:
                out = F.relu(out)
                if self.p > 0.0:
                    keep = dropout_keep_mask(out.numel(), self.seed, offsets[i], self.p).reshape(out.shape)
                    out = out * torch.from_numpy(keep).to(out.dtype) / (1.0 - self.p)
            out = rb(out)
            saved.append((agg, a_t, out, last))
            h = out
        self._saved = saved
        return h

    def backward(self, grad_logits):
        g = rb(grad_logits)
        grads_w = [None] * len(self.weights)
        for i in reversed(range(len(self.weights))):
            agg, a_t, out, last = self._saved[i]
            w = rb(self.weights[i].reshape(self.dims[i], self.dims[i + 1]))
            if not last:
                g = g * (out > 0).to(g.dtype)
                scale = 1.0 / (1.0 - self.p) if self.p > 0.0 else 1.0
            else:
                scale = 1.0
            grads_w[i] = (scale * torch.mm(torch.t(agg), g)).reshape(-1)
            grad_agg = rb(scale * torch.mm(g, torch.t(w)))
            g = rb(torch.sparse.mm(a_t, grad_agg))
        return g, grads_w


def train_epochs_bf16(x0, weights, dims, adj_shards, labels, num_nodes, num_classes, epochs=10, lr=3e-3, dropout_p=0.0,
                      seed=0, offsets_of_epoch=None):
    """The epoch loop of train_epochs (examples/train.py:83-112,164-193) over the bf16-storage network: the trained
    tensors (weights, input features) stay in the working precision, the network reads their bf16 roundings, the
    gradient of the features arrives rounded to bf16, the weight gradients do not.  ``offsets_of_epoch(e)`` gives the
    dropout offsets of the layers in epoch e.
    """
    net = OracleNetBf16(weights, dims, dropout_p=dropout_p, seed=seed)
    x = x0.clone().reshape(-1)
    state = {}
    losses = []
    for e in range(epochs):
        offsets = offsets_of_epoch(e) if offsets_of_epoch is not None else None
        logits = net.forward(x, adj_shards, offsets)
        loss, softmax, onehot = cross_entropy_forward(logits, labels, num_nodes, num_classes)
        g = cross_entropy_backward(softmax, onehot.to(softmax.dtype), num_nodes)
        gx, gws = net.backward(g)
        adamw_step(net.weights + [x], gws + [gx.reshape(-1)], state, lr=lr)
        losses.append(float(loss))
    return losses, x, net.weights
