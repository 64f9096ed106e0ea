"""Synthetic graphs and features of the benchmark configurations.

The reference trains on downloaded datasets preprocessed by plexus/utils/dataset.py (GCN
normalisation :101, random vertex permutation :128-243) and loaded per rank as a CSR block plus the CSR
of its transpose (plexus/utils/dataloader.py:343-368).  There is no network here, so graphs of the same
shape are generated: uniform random, R-MAT and Chung-Lu power-law graphs, symmetrised, with self
loops, GCN-normalised, randomly permuted, and cut into a rank's block where asked.  Everything is
plain torch on one device (the GPU for the full-size configurations) and is seeded through a
``torch.Generator`` of that device.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass
class Graph:
    """A (block of a) normalised adjacency matrix in CSR form and the CSR of its transpose."""

    shape: Tuple[int, int]
    rowptr: torch.Tensor  # int64 [M + 1]
    col: torch.Tensor  # int64 [nnz]
    val: torch.Tensor  # fp32  [nnz]
    rowptr_t: torch.Tensor
    col_t: torch.Tensor
    val_t: torch.Tensor

    @property
    def nnz(self) -> int:
        return int(self.col.numel())

    def torch_csr(self, transpose: bool = False) -> torch.Tensor:
        if transpose:
            return torch.sparse_csr_tensor(self.rowptr_t, self.col_t, self.val_t, size=(self.shape[1], self.shape[0]))
        return torch.sparse_csr_tensor(self.rowptr, self.col, self.val, size=self.shape)

    def degree_stats(self):
        deg = self.rowptr[1:] - self.rowptr[:-1]
        return {"rows": self.shape[0], "cols": self.shape[1], "nnz": self.nnz, "max_row_nnz": int(deg.max()) if deg.numel() else 0,
                "mean_row_nnz": float(self.nnz) / max(self.shape[0], 1)}


def _gen(seed: int, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def uniform_pairs(n: int, n_pairs: int, gen: torch.Generator, device) -> Tuple[torch.Tensor, torch.Tensor]:
    src = torch.randint(0, n, (n_pairs,), generator=gen, device=device, dtype=torch.int64)
    dst = torch.randint(0, n, (n_pairs,), generator=gen, device=device, dtype=torch.int64)
    return src, dst


def rmat_pairs(n: int, n_pairs: int, gen: torch.Generator, device, a=0.57, b=0.19, c=0.19) -> Tuple[torch.Tensor, torch.Tensor]:
    """R-MAT (Chakrabarti et al.) pairs over ceil(log2 n) bit levels; ids >= n are rejected."""
    scale = max(1, math.ceil(math.log2(max(n, 2))))
    src = torch.zeros(n_pairs, dtype=torch.int64, device=device)
    dst = torch.zeros(n_pairs, dtype=torch.int64, device=device)
    for _ in range(scale):
        u = torch.rand(n_pairs, generator=gen, device=device)
        src_bit = u >= (a + b)
        dst_bit = ((u >= a) & (u < a + b)) | (u >= a + b + c)
        src = (src << 1) | src_bit.to(torch.int64)
        dst = (dst << 1) | dst_bit.to(torch.int64)
    keep = (src < n) & (dst < n)
    return src[keep], dst[keep]


def chung_lu_pairs(n: int, n_pairs: int, gen: torch.Generator, device, gamma: float = 2.1) -> Tuple[torch.Tensor, torch.Tensor]:
    """Chung-Lu pairs: both endpoints drawn with probability proportional to (i + 1)^(-1 / (gamma - 1))."""
    alpha = 1.0 / (gamma - 1.0)
    w = torch.arange(1, n + 1, dtype=torch.float64, device=device).pow(-alpha)
    cdf = torch.cumsum(w, 0)
    cdf = cdf / cdf[-1]
    u = torch.rand(2 * n_pairs, generator=gen, device=device, dtype=torch.float64)
    ids = torch.searchsorted(cdf, u).clamp_(max=n - 1)
    return ids[:n_pairs], ids[n_pairs:]


def _undirected_keys(src, dst, n: int) -> torch.Tensor:
    """Sorted unique keys lo * n + hi of the non-loop pairs."""
    lo = torch.minimum(src, dst)
    hi = torch.maximum(src, dst)
    keep = lo != hi
    return torch.unique(lo[keep] * n + hi[keep])


def build_graph(
    n: int,
    kind: str,
    target_undirected: int,
    seed: int = 0,
    device="cpu",
    permute: bool = True,
    double_perm: bool = False,
    block: Optional[Tuple[Tuple[int, int], Tuple[int, int]]] = None,
    exact_pairs: Optional[int] = None,
    **kind_args,
) -> Graph:
    """Generate, symmetrise, add self loops, GCN-normalise, permute, and (optionally) cut a block.

    ``kind`` is "uniform", "rmat" or "chunglu".  Pairs are drawn until ``target_undirected`` distinct
    undirected non-loop edges exist (``exact_pairs`` draws that many pairs once instead, whatever the
    number of distinct edges).  The normalisation is D^-1/2 (A + I) D^-1/2 with unit edge weights, i.e.
    value 1 / sqrt(d_i d_j) with d the row count including the self loop.  With ``permute`` the vertices
    are renumbered by a random permutation (rows and columns alike); with ``double_perm`` rows and
    columns get two different permutations, as in plexus/utils/dataset.py:130-198.  ``block`` =
    ((r0, r1), (c0, c1)) keeps that block re-based to zero as plexus/utils/dataloader.py:343-361 does.
    """
    gen = _gen(seed, device)
    draw = {"uniform": uniform_pairs, "rmat": rmat_pairs, "chunglu": chung_lu_pairs}[kind]
    if exact_pairs is not None:
        s, d = draw(n, exact_pairs, gen, device, **kind_args)
        keys = _undirected_keys(s, d, n)
    else:
        keys = torch.empty(0, dtype=torch.int64, device=device)
        rounds = 0
        while keys.numel() < target_undirected and rounds < 64:
            want = max(int((target_undirected - keys.numel()) * 1.25), 1024)
            s, d = draw(n, want, gen, device, **kind_args)
            keys = torch.unique(torch.cat([keys, _undirected_keys(s, d, n)]))
            del s, d
            rounds += 1
        if keys.numel() > target_undirected:
            # drop a uniformly random surplus so that the edge count is the one asked for
            drop = torch.randperm(keys.numel(), generator=gen, device=device)[: keys.numel() - target_undirected]
            mask = torch.ones(keys.numel(), dtype=torch.bool, device=device)
            mask[drop] = False
            keys = keys[mask]
    lo = keys // n
    hi = keys % n
    del keys
    # degrees include the self loop; the graph is symmetric
    deg = torch.bincount(torch.cat([lo, hi]), minlength=n) + 1
    dinv = deg.to(torch.float64).pow(-0.5)
    loops = torch.arange(n, dtype=torch.int64, device=device)
    row = torch.cat([lo, hi, loops])
    col = torch.cat([hi, lo, loops])
    del lo, hi
    val = (dinv[row] * dinv[col]).to(torch.float32)

    if permute:
        p_row = torch.randperm(n, generator=gen, device=device)
        p_col = torch.randperm(n, generator=gen, device=device) if double_perm else p_row
        row = p_row[row]
        col = p_col[col]

    shape = (n, n)
    if block is not None:
        (r0, r1), (c0, c1) = block
        keep = (row >= r0) & (row < r1) & (col >= c0) & (col < c1)
        row = row[keep] - r0
        col = col[keep] - c0
        val = val[keep]
        shape = (r1 - r0, c1 - c0)

    rowptr, col_s, val_s = coo_to_csr(row, col, val, shape)
    rowptr_t, col_t, val_t = coo_to_csr(col, row, val, (shape[1], shape[0]))
    return Graph(shape, rowptr, col_s, val_s, rowptr_t, col_t, val_t)


def coo_to_csr(row, col, val, shape):
    """Sort distinct (row, col) entries into CSR order; returns (rowptr int64, col int64, val)."""
    m, k = shape
    order = torch.argsort(row * k + col)
    counts = torch.bincount(row, minlength=m)
    rowptr = torch.zeros(m + 1, dtype=torch.int64, device=row.device)
    torch.cumsum(counts, 0, out=rowptr[1:])
    return rowptr, col[order].contiguous(), val[order].contiguous()


# ---------------------------------------------------------------------------------------------
# the benchmark configurations (sizes can be scaled down for tests)
# ---------------------------------------------------------------------------------------------
def config1(device="cpu", seed=0):
    """2,708 nodes, 10,556 uniform directed pairs symmetrised; X 2,708 x 1,433 Bernoulli(0.013); 7 classes."""
    n = 2708
    g = build_graph(n, "uniform", 0, seed=seed, device=device, permute=False, exact_pairs=10556)
    gen = _gen(seed + 1, device)
    x = (torch.rand(n, 1433, generator=gen, device=device) < 0.013).to(torch.float32)
    y = torch.randint(0, 7, (n,), generator=gen, device=device, dtype=torch.int64)
    return g, x, y, [1433, 16, 7]


def glorot_weights(dims, seed=0):
    """Glorot-uniform (in, out) matrices drawn on the host generator, returned flat."""
    gen = torch.Generator().manual_seed(seed)
    out = []
    for i in range(len(dims) - 1):
        bound = math.sqrt(6.0 / (dims[i] + dims[i + 1]))
        w = (torch.rand(dims[i], dims[i + 1], generator=gen, dtype=torch.float64) * 2 - 1) * bound
        out.append(w.to(torch.float32).reshape(-1))
    return out


def config2_graph(device, seed=0, scale=1.0):
    """R-MAT(0.57, 0.19, 0.19, 0.05), N = 232,965, about 114.6 M stored entries with self loops."""
    n = max(64, int(232965 * scale))
    target_nnz = int(114.6e6 * scale)
    return build_graph(n, "rmat", (target_nnz - n) // 2, seed=seed, device=device)


def config3_graph(device, seed=0, scale=1.0):
    """Chung-Lu, exponent 2.1, N = 2,449,029, about 123.7 M symmetrised edges plus self loops."""
    n = max(64, int(2449029 * scale))
    target_undirected = int(123.7e6 * scale) // 2
    return build_graph(n, "chunglu", target_undirected, seed=seed, device=device, gamma=2.1)


def config4_block(device, seed=0, scale=1.0):
    """One rank's block of a 2 x 2 x 2 grid: rows and columns [0, N/2) of a doubly permuted R-MAT graph."""
    n = max(128, int(8388608 * scale))
    n -= n % 2
    target_nnz = int(256e6 * scale)
    half = n // 2
    return build_graph(n, "rmat", (target_nnz - n) // 2, seed=seed, device=device, double_perm=True,
                       block=((0, half), (0, half)))


def normal_features(rows, cols, device, seed=0, dtype=torch.float32):
    gen = _gen(seed + 17, device)
    return torch.randn(rows, cols, generator=gen, device=device, dtype=torch.float32).to(dtype)


def uniform_labels(rows, classes, device, seed=0):
    gen = _gen(seed + 29, device)
    return torch.randint(0, classes, (rows,), generator=gen, device=device, dtype=torch.int64)
