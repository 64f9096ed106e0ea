"""Graph preprocessing on the device and the 2-D partition files.

Counterpart of plexus/utils/dataset.py: GCN normalisation (:101), the random vertex permutation(s)
written there as sparse products P.A.P2^T (:128-243), the degree-bucket labels of unlabelled graphs
(:104-116) and ``partition_graph_2d`` (:368-543) with the same directory layout:

    metadata.pt                      (num_nodes, num_features, num_classes)
    edge_index/{0,1}/{i}_{j}.pt      (int64 [2, E_ij] with GLOBAL vertex ids, fp32 [E_ij])
    input_features/{i}_{j}.pt        fp32 [rows of node chunk i, columns of feature chunk j]
    output_labels/{0,1}/{i}.pt       int64 [rows of node chunk i]

``{0,1}`` is the first / second permutation of a doubly permuted graph.  Every file is a plain tensor or
a tuple of tensors / ints, so ``torch.load(..., weights_only=True)`` reads files written by either side.

The reference's *unpartitioned* file is a pickled ``torch_geometric.data.Data`` object (:241); that class
is not available here and unpickling it would execute code from the file, so only the partitioned layout is
read and written.  Datasets are not downloaded: the entry point takes the edge list, features and labels
as tensors.

The sorting, CSR building, transposition, normalisation and relabelling run in libplexus_hip on the GPU;
torch is used for concatenation, slicing and file I/O.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Optional

import torch

from .. import ops
from .general import pad_dimension


@dataclass
class ProcessedGraph:
    """The fields of the object that ``preprocess_graph`` saves in the reference (dataset.py:241)."""

    edge_index: torch.Tensor  # int64 [2, E], sorted by (row, col)
    edge_weight: torch.Tensor  # fp32 [E]
    x: torch.Tensor  # fp32 [N, F], rows in the order of the columns of edge_index
    y: torch.Tensor  # int64 [N], rows in the order of the rows of edge_index
    num_classes: int
    edge_index_2: Optional[torch.Tensor] = None  # second adjacency of the double permutation (odd layers)
    edge_weight_2: Optional[torch.Tensor] = None
    y_2: Optional[torch.Tensor] = None

    @property
    def num_nodes(self) -> int:
        return int(self.x.shape[0])

    @property
    def double_perm(self) -> bool:
        return self.edge_index_2 is not None


def normalize_features(x: torch.Tensor) -> torch.Tensor:
    """Rows divided by their sum clamped to >= 1 (T.NormalizeFeatures, applied at dataset.py:56-67,96)."""
    return x / x.sum(dim=-1, keepdim=True).clamp_(min=1.0)


def gcn_norm(edge_index: torch.Tensor, edge_weight: Optional[torch.Tensor], num_nodes: int, directed: bool = False) -> ops.CsrMatrix:
    """D^-1/2 (A + I) D^-1/2 as a CSR matrix on the device, d = weighted in-degree (sum over the edges that
    point at a vertex, self loop included), as T.GCNNorm computes it (dataset.py:101).

    With ``directed`` the result is the transpose, which the reference aggregates with for directed graphs
    (dataset.py:166-168).  Duplicate edges are summed, as the CSR conversion of :158-160 does."""
    return ops.gcn_norm_from_edges(edge_index, edge_weight, num_nodes, transposed=directed)


def degree_bucket_labels(edge_index: torch.Tensor, num_nodes: int, num_classes: int) -> torch.Tensor:
    """Labels of an unlabelled graph: vertices sorted by out-edge count and cut into ``num_classes`` nearly
    equal buckets (dataset.py:104-116, numpy.array_split sizes).  Ties are ordered by vertex id (stable sort);
    the reference's unstable argsort leaves their order open."""
    counts = torch.bincount(edge_index[0], minlength=num_nodes)
    order = torch.argsort(counts, stable=True)
    base, extra = divmod(num_nodes, num_classes)
    sizes = torch.tensor([base + 1 if i < extra else base for i in range(num_classes)], device=order.device)
    bucket_of_rank = torch.repeat_interleave(torch.arange(num_classes, device=order.device), sizes)
    y = torch.empty(num_nodes, dtype=torch.int64, device=order.device)
    y[order] = bucket_of_rank
    return y


def permute_adjacency(adj: ops.CsrMatrix, perm_rows: torch.Tensor, perm_cols: torch.Tensor, adj_t: Optional[ops.CsrMatrix] = None):
    """(edge_index, edge_weight) of P_rows . A . P_cols^T with P[i, perm[i]] = 1, i.e. entry (i, j) of the result
    is entry (perm_rows[i], perm_cols[j]) of A (dataset.py:137-216), sorted by (row, col).  ``adj_t`` is the CSR of
    A^T, which the permutation works from; give it when one matrix is permuted more than once."""
    return ops.csr_to_edges(ops.csr_permute(adj, perm_rows, perm_cols, a_t=adj_t))


def preprocess_graph(
    edge_index: torch.Tensor,
    edge_weight: Optional[torch.Tensor],
    x: Optional[torch.Tensor],
    y: Optional[torch.Tensor],
    num_classes: int,
    double_perm: bool = True,
    directed: bool = False,
    num_features: int = 128,
    generator: Optional[torch.Generator] = None,
    perm: Optional[torch.Tensor] = None,
    perm2: Optional[torch.Tensor] = None,
    num_nodes: Optional[int] = None,
) -> ProcessedGraph:
    """The body of ``preprocess_graph`` (dataset.py:86-243) from tensors instead of a downloaded dataset.

    Missing features are drawn uniform and row-normalised, missing labels are degree buckets
    (the ``unsupervised`` case, :90-116); the adjacency is GCN-normalised, then both it, the features and the
    labels are permuted: A = P.A.P2^T, x = x[perm2], y = y[perm], and for the double permutation also
    A2 = P2.A.P^T and y_2 = y[perm2].  Without ``double_perm`` P2 = P.  The permutations are drawn on the host
    generator as the reference does (:130-133) unless they are passed in.
    """
    dev = edge_index.device
    n = int(num_nodes if num_nodes is not None else (x.shape[0] if x is not None else int(edge_index.max()) + 1))
    if x is None:
        x = normalize_features(torch.rand(n, num_features, generator=generator).to(dev))
    adj = gcn_norm(edge_index, edge_weight, n, directed=directed)
    adj_t = ops.csr_transpose(adj)  # both permutations below work from it
    if y is None:
        ei_norm, _ = ops.csr_to_edges(adj if not directed else adj_t)
        y = degree_bucket_labels(ei_norm, n, num_classes)
    y = torch.nan_to_num(y.reshape(-1).to(torch.float64), nan=-1.0).to(torch.int64) if y.is_floating_point() else y.reshape(-1).to(torch.int64)
    if perm is None:
        perm = torch.randperm(n, generator=generator)
    if double_perm and perm2 is None:
        perm2 = torch.randperm(n, generator=generator)
    perm = perm.to(dev)
    p_cols = perm2.to(dev) if double_perm else perm
    ei, w = permute_adjacency(adj, perm, p_cols, adj_t)
    out = ProcessedGraph(edge_index=ei, edge_weight=w, x=x.to(dev)[p_cols, :], y=y.to(dev)[perm], num_classes=int(num_classes))
    if double_perm:
        out.edge_index_2, out.edge_weight_2 = permute_adjacency(adj, p_cols, perm, adj_t)
        out.y_2 = y.to(dev)[p_cols]
    return out


def partition_graph_2d(graph: ProcessedGraph, num_partitions: int, output_dir: str) -> None:
    """Write the 2-D partition files of dataset.py:368-543 (layout in the module docstring).

    Node chunk i is rows [i * c, min((i + 1) * c, N)) with c = pad(N, P) / P; an adjacency file holds the
    edges whose row lies in chunk i and whose column lies in chunk j, with global ids; a feature file holds node
    chunk i x feature chunk j; label files exist per node chunk."""
    n, f = int(graph.x.shape[0]), int(graph.x.shape[1])
    p = int(num_partitions)
    chunk_nodes = pad_dimension(n, p) // p
    chunk_feats = pad_dimension(f, p) // p
    os.makedirs(output_dir, exist_ok=True)
    torch.save((n, f, int(graph.num_classes)), os.path.join(output_dir, "metadata.pt"))
    adjs = [(graph.edge_index, graph.edge_weight)]
    labels = [graph.y]
    if graph.double_perm:
        adjs.append((graph.edge_index_2, graph.edge_weight_2))
        labels.append(graph.y_2)
    for k in range(len(adjs)):
        os.makedirs(os.path.join(output_dir, "edge_index", str(k)), exist_ok=True)
        os.makedirs(os.path.join(output_dir, "output_labels", str(k)), exist_ok=True)
    os.makedirs(os.path.join(output_dir, "input_features"), exist_ok=True)
    for i in range(p):
        r0, r1 = i * chunk_nodes, min((i + 1) * chunk_nodes, n)
        for k, (ei, w) in enumerate(adjs):
            in_rows = (ei[0] >= r0) & (ei[0] < r1)
            ei_rows, w_rows = ei[:, in_rows], w[in_rows]  # one pass over all edges per row chunk, then per block
            for j in range(p):
                c0, c1 = j * chunk_nodes, min((j + 1) * chunk_nodes, n)
                m = (ei_rows[1] >= c0) & (ei_rows[1] < c1)
                torch.save((ei_rows[:, m].cpu().clone(), w_rows[m].cpu().clone()),
                           os.path.join(output_dir, "edge_index", str(k), "%d_%d.pt" % (i, j)))
            torch.save(labels[k][r0:r1].cpu().clone(), os.path.join(output_dir, "output_labels", str(k), "%d.pt" % i))
        for j in range(p):
            f0, f1 = j * chunk_feats, min((j + 1) * chunk_feats, f)
            torch.save(graph.x[r0:r1, f0:f1].cpu().clone(), os.path.join(output_dir, "input_features", "%d_%d.pt" % (i, j)))
