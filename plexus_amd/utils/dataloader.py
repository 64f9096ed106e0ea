"""Loader of the 2-D partition files: one rank's adjacency blocks, feature slab and labels, built on the GPU.

Counterpart of plexus/utils/dataloader.py.  The index arithmetic (which rows, columns, features and labels a
rank of a G_x x G_y x G_z grid owns, which partition files cover them, how the slabs are padded and
flattened) follows the reference line by line in meaning; the work differs: the files that cover a shard are
concatenated on the device and ``plx_coo_block_to_csr_f32`` / ``plx_csr_transpose_f32`` cut, re-base, sort and
transpose them there, where the reference builds two CSR tensors on the host per shard (:343-375).

Only partitioned directories are read (``metadata.pt`` present): the unpartitioned file is a pickled
third-party object.  Files are read with ``torch.load(..., weights_only=True)``.

The grid defaults to 1 x 1 x 1, the only one the layers run on here; other grids and ranks can be named to
cut the share of one rank of a larger job at its real shape.
"""
from __future__ import annotations

import glob
import os
from typing import Sequence

import torch
import torch.nn.functional as F

from .. import ops
from .general import pad_dimension


class DataLoader:
    def __init__(self, data_dir: str, num_gcn_layers: int, grid: Sequence[int] = (1, 1, 1), ranks: Sequence[int] = (0, 0, 0),
                 device="cuda"):
        """``grid`` = (G_intra_r, G_intra_c, G_intra_d) and ``ranks`` = (row, column, depth) rank, the quantities the
        reference reads from its communication handle (plexus/utils/general.py:37-48)."""
        self.data_dir = data_dir
        self.num_gcn_layers = int(num_gcn_layers)
        self.device = torch.device(device)
        # the reference orders the three groups ("z", "x", "y") = (depth, row, column): dataloader.py:57
        self._num_gpus = [int(grid[2]), int(grid[0]), int(grid[1])]
        self._ranks = [int(ranks[2]), int(ranks[0]), int(ranks[1])]
        for g, r in zip(self._num_gpus, self._ranks):
            if g < 1 or not 0 <= r < g:
                raise ValueError("rank %d outside a group of %d" % (r, g))
        self.partitioned = os.path.exists(os.path.join(data_dir, "metadata.pt"))
        if not self.partitioned:
            raise ValueError("%s holds no metadata.pt: only 2-D partitioned directories are read" % data_dir)
        self.double_perm = os.path.exists(os.path.join(data_dir, "edge_index", "1"))
        self.labels_dir = os.path.join(data_dir, "output_labels")
        self.num_partitions_dim = len(glob.glob(os.path.join(self.labels_dir, "0", "*.pt")))
        if self.num_partitions_dim < 1:
            raise ValueError("%s holds no label partitions" % self.labels_dir)
        self.adj_dir = os.path.join(data_dir, "edge_index")
        self.features_dir = os.path.join(data_dir, "input_features")

    # ---- which indices this rank owns (dataloader.py:47-151) ----
    def _set_graph_attributes(self):
        meta = torch.load(os.path.join(self.data_dir, "metadata.pt"), weights_only=True)
        self.num_nodes, self.num_features, self.num_classes = (int(v) for v in meta)
        num_gpus, ranks = self._num_gpus, self._ranks
        nodes_step = pad_dimension(self.num_nodes, num_gpus[1]) // num_gpus[1]
        feats_step = pad_dimension(self.num_features, num_gpus[2], num_gpus[0]) // num_gpus[2]
        self.nodes_start, self.nodes_stop = ranks[1] * nodes_step, (ranks[1] + 1) * nodes_step
        self.features_start, self.features_stop = ranks[2] * feats_step, (ranks[2] + 1) * feats_step
        depth_step = pad_dimension(nodes_step * feats_step, num_gpus[0]) // num_gpus[0]
        self.depth_start, self.depth_stop = ranks[0] * depth_step, (ranks[0] + 1) * depth_step
        # the group that splits the rows of the last layer's output holds the labels (:90-106)
        labels_group = {1: 0, 2: 2, 0: 1}[self.num_gcn_layers % 3]
        labels_step = pad_dimension(self.num_nodes, num_gpus[labels_group]) // num_gpus[labels_group]
        self.labels_start, self.labels_stop = ranks[labels_group] * labels_step, (ranks[labels_group] + 1) * labels_step
        # block of the adjacency matrix per layer position, cycling with period 3 (:111-151)
        self.adj_rows, self.adj_cols = [], []
        for i in range(min(3, self.num_gcn_layers)):
            g1, g2 = [(0, 1), (2, 0), (1, 2)][i]
            step1 = pad_dimension(self.num_nodes, num_gpus[g1]) // num_gpus[g1]
            step2 = pad_dimension(self.num_nodes, num_gpus[g2]) // num_gpus[g2]
            self.adj_rows.append((ranks[g1] * step1, (ranks[g1] + 1) * step1))
            self.adj_cols.append((ranks[g2] * step2, (ranks[g2] + 1) * step2))

    def _partition_range(self, start, stop, size):
        """Indices of the partition files that cover [start, stop) (:176-199 and alike)."""
        p = self.num_partitions_dim
        return range(min(start // size, p), min((stop - 1) // size + 1, p))

    # ---- adjacency (:153-213, :327-375) ----
    def _load_adj_shard(self, layer_num):
        size = pad_dimension(self.num_nodes, self.num_partitions_dim) // self.num_partitions_dim
        (r0, r1), (c0, c1) = self.adj_rows[layer_num % 3], self.adj_cols[layer_num % 3]
        adj_num = 1 if (self.double_perm and layer_num % 2 != 0) else 0
        idx, val = [], []
        for i in self._partition_range(r0, r1, size):
            for j in self._partition_range(c0, c1, size):
                ei, w = torch.load(os.path.join(self.adj_dir, str(adj_num), "%d_%d.pt" % (i, j)), weights_only=True)
                idx.append(ei.to(torch.int64))
                val.append(w.to(torch.float32))
        if idx:
            ei = torch.cat(idx, dim=1).to(self.device)
            w = torch.cat(val).to(self.device)
        else:
            ei = torch.empty((2, 0), dtype=torch.int64, device=self.device)
            w = torch.empty(0, dtype=torch.float32, device=self.device)
        # mask to the block, re-base, CSR and CSR of the transpose -- on the device
        return ops.csr_pair_from_edges(ei, w, (self.num_nodes, self.num_nodes), (r0, r1), (c0, c1))

    # ---- features (:215-270, :377-424) ----
    def _load_features(self):
        p = self.num_partitions_dim
        size1 = pad_dimension(self.num_nodes, p) // p
        size2 = pad_dimension(self.num_features, p) // p
        part_nodes_start = (self.nodes_start // size1) * size1
        part_feats_start = (self.features_start // size2) * size2
        rows = []
        for i in self._partition_range(self.nodes_start, self.nodes_stop, size1):
            cols = [torch.load(os.path.join(self.features_dir, "%d_%d.pt" % (i, j)), weights_only=True)
                    for j in self._partition_range(self.features_start, self.features_stop, size2)]
            if cols:
                rows.append(torch.cat(cols, dim=1))
        want_rows, want_cols = self.nodes_stop - self.nodes_start, self.features_stop - self.features_start
        if rows:
            merged = torch.cat(rows, dim=0)
            local = merged[self.nodes_start - part_nodes_start: self.nodes_stop - part_nodes_start,
                           self.features_start - part_feats_start: self.features_stop - part_feats_start]
        else:
            local = torch.zeros(want_rows, want_cols)
        local = F.pad(local.to(torch.float32), (0, want_cols - local.shape[1], 0, want_rows - local.shape[0]))
        # the depth group splits the flattened slab (its length is a multiple of the group size by construction)
        return local.reshape(-1)[self.depth_start: self.depth_stop].to(self.device).requires_grad_()

    # ---- labels (:272-325, :426-452) ----
    def _load_labels(self):
        p = self.num_partitions_dim
        size = pad_dimension(self.num_nodes, p) // p
        part_start = (self.labels_start // size) * size
        labels_num = 1 if (self.double_perm and self.num_gcn_layers % 2 == 0) else 0
        parts = [torch.load(os.path.join(self.labels_dir, str(labels_num), "%d.pt" % i), weights_only=True)
                 for i in self._partition_range(self.labels_start, self.labels_stop, size)]
        merged = torch.cat(parts) if parts else torch.empty(0, dtype=torch.int64)
        local = merged[self.labels_start - part_start: self.labels_stop - part_start]
        local = F.pad(local, (0, (self.labels_stop - self.labels_start) - local.shape[0])).to(torch.int64)
        return local.to(self.device)

    def load(self):
        """(adj_shards, input_features, output_labels, num_nodes, num_features, num_classes) as dataloader.py:454-540.

        ``adj_shards[i]`` = (A, A^T) of layer position i as ``plexus_amd.ops.CsrMatrix`` objects (the layers accept
        them in place of torch CSR tensors); there are min(3, layers) of them, min(6, layers) for a doubly
        permuted graph, whose odd positions use the second adjacency."""
        with torch.no_grad():
            self._set_graph_attributes()
            n_shards = min(6 if self.double_perm else 3, self.num_gcn_layers)
            adj_shards = [self._load_adj_shard(i) for i in range(n_shards)]
            features = self._load_features()
            labels = self._load_labels()
        return adj_shards, features, labels, self.num_nodes, self.num_features, self.num_classes
