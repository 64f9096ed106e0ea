"""Tensor-level front end of the C ABI: argument checks, output allocation, stream plumbing.

PyTorch is used for device memory and streams only; every computation below is a call into
libplexus_hip.so on the current HIP stream.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from . import _lib
from ._lib import PLX_GEMM_DROPOUT, PLX_GEMM_RELU, check


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise _lib.PlexusHipError(
                "plexus_amd runs on the GPU only: got a tensor on %s (there is no CPU path)" % t.device
            )


def _rowmajor(t: torch.Tensor) -> torch.Tensor:
    """A 2-D tensor whose rows are contiguous (any row pitch); copies only if it has to."""
    if t.dim() != 2:
        raise ValueError("expected a 2-D tensor, got shape %s" % (tuple(t.shape),))
    if t.stride(1) != 1 and t.shape[1] > 1:
        return t.contiguous()
    if t.shape[1] == 1 and t.stride(0) < 1:
        return t.contiguous()
    if t.shape[0] > 1 and t.stride(0) < t.shape[1]:
        return t.contiguous()
    return t


def _need_fp32(who: str, **tensors) -> None:
    """The fp32 entry points read raw pointers: anything but float32 would be misread without an error."""
    for name, t in tensors.items():
        if t is not None and t.dtype != torch.float32:
            raise TypeError("%s: %s must be float32, got %s" % (who, name, t.dtype))


def _ld(t: torch.Tensor) -> int:
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)


class CsrMatrix:
    """A CSR matrix prepared for the SpMM kernel: int32 indices, fp32 values and the row plan.

    Built from a torch sparse-CSR tensor (``from_torch``) or from raw arrays.  The plan (row binning
    and the split of long rows into segments) is computed once (with ``defer_plan``: at the first
    product); the int32 arrays are owned here and outlive it.  The scratch of the products is cached on the object, so products of one matrix must
    be ordered (one stream, or events between streams); different matrices are independent.
    """

    def __init__(self, rowptr: torch.Tensor, col: torch.Tensor, val: torch.Tensor, shape, seg_len: int = 0,
                 defer_plan: bool = False):
        _need_gpu(rowptr, col, val)
        m, k = int(shape[0]), int(shape[1])
        nnz = int(col.numel())
        if rowptr.numel() != m + 1:
            raise ValueError("rowptr has %d entries for %d rows" % (rowptr.numel(), m))
        if val.numel() != nnz:
            raise ValueError("col and val differ in length")
        lib = _lib.load()
        if rowptr.dtype == torch.int64 or col.dtype == torch.int64:
            if nnz >= 2**31 or max(m, k) >= 2**31 - 1:
                raise ValueError("matrix too large for int32 indexing")
            rp64 = rowptr.to(torch.int64).contiguous()
            ci64 = col.to(torch.int64).contiguous()
            rp32 = torch.empty(m + 1, dtype=torch.int32, device=val.device)
            ci32 = torch.empty(nnz, dtype=torch.int32, device=val.device)
            check(
                lib.plx_csr_narrow_i64(m, nnz, rp64.data_ptr(), ci64.data_ptr(), rp32.data_ptr(), ci32.data_ptr(), _stream()),
                "plx_csr_narrow_i64",
            )
            rowptr, col = rp32, ci32
        self.rowptr = rowptr.to(torch.int32).contiguous()
        self.col = col.to(torch.int32).contiguous()
        self.val = val.to(torch.float32).contiguous()
        self.shape = (m, k)
        self.nnz = nnz
        self.device = val.device
        self._seg_len = int(seg_len)
        self._plan_handle = None
        self._ws: Optional[torch.Tensor] = None
        if not defer_plan:
            self.prepare()  # checks the arrays too: a malformed matrix is refused here, not at its first product

    @classmethod
    def from_torch(cls, a: torch.Tensor, seg_len: int = 0) -> "CsrMatrix":
        if a.layout != torch.sparse_csr:
            raise ValueError("expected a sparse CSR tensor, got layout %s" % a.layout)
        return cls(a.crow_indices(), a.col_indices(), a.values(), a.shape, seg_len)

    def prepare(self) -> "CsrMatrix":
        """Build the row plan now (it allocates and waits for the device, so not under stream capture)."""
        self._plan
        return self

    @property
    def _plan(self):
        """The row plan of the products (bins, segments, hub tables).  The builders of this module hand out
        matrices whose arrays are well-formed by construction and defer it to the first product, so that a
        matrix that is only converted or transposed never pays for it."""
        if self._plan_handle is None:
            handle = _lib.C.c_void_p()
            m, k = self.shape
            check(
                _lib.load().plx_spmm_plan_create(
                    _lib.C.byref(handle), m, k, self.nnz, self.rowptr.data_ptr(), self.col.data_ptr() if self.nnz else None,
                    self._seg_len, _stream(),
                ),
                "plx_spmm_plan_create",
            )
            self._plan_handle = handle
        return self._plan_handle

    def __del__(self):
        plan = getattr(self, "_plan_handle", None)
        if plan is not None and plan.value:
            try:
                _lib.load().plx_spmm_plan_destroy(plan)
            except Exception:
                pass
            self._plan_handle = None

    @property
    def n_long_rows(self) -> int:
        return int(_lib.load().plx_spmm_plan_info(self._plan, 3))

    @property
    def n_segments(self) -> int:
        return int(_lib.load().plx_spmm_plan_info(self._plan, 4))

    def size(self, dim: int) -> int:
        return self.shape[dim]

    def set_slicing(self, mode: int) -> None:
        """Column slicing of H in the products of this matrix: 0 = where the library's rule says so (the default),
        1 = whenever a row of H exceeds 256 bytes, -1 = never.  The result of a product does not depend on how it was
        sliced, only on the mode."""
        check(_lib.load().plx_spmm_plan_set_slicing(self._plan, int(mode)), "plx_spmm_plan_set_slicing")

    @property
    def n_hub_rows(self) -> int:
        """Rows taken by the hub pass (0: this matrix has no hub tables)."""
        return int(_lib.load().plx_spmm_plan_info(self._plan, 6))

    @property
    def hub_entries(self) -> int:
        return int(_lib.load().plx_spmm_plan_info(self._plan, 7))

    @property
    def hub_table_bytes(self) -> int:
        """Device memory the plan holds for the hub pass (the streams: 5 bytes per stored entry), 0 without one."""
        return max(0, int(_lib.load().plx_spmm_plan_info(self._plan, 8)))

    def build_hub(self) -> None:
        """Builds the tables of the hub pass whatever the library's size rule says (it builds them by itself for large
        power-law matrices): the longest rows then walk the columns together, sharing the rows of H through L2."""
        check(_lib.load().plx_spmm_plan_build_hub(self._plan, _stream()), "plx_spmm_plan_build_hub")
        self._ws = None

    def build_hub_wide(self) -> None:
        """Builds the hub tables in the layout for bf16 rows of 512 bytes and more (256 columns per tile, half as many
        sums per wavefront).  The front end does this by itself before the first such product of a matrix that has the
        regular tables."""
        check(_lib.load().plx_spmm_plan_build_hub_wide(self._plan, _stream()), "plx_spmm_plan_build_hub_wide")
        self._wide_tried = True
        self._ws = None

    @property
    def n_hub_rows_wide(self) -> int:
        return int(_lib.load().plx_spmm_plan_info(self._plan, 9))

    def set_hub(self, mode: int) -> None:
        """0 = products use the hub pass where the tables exist and the operands allow it (the default), -1 = never.
        With and without the pass a product agrees to fp32 rounding, not bit for bit."""
        check(_lib.load().plx_spmm_plan_set_hub(self._plan, int(mode)), "plx_spmm_plan_set_hub")
        self._ws = None

    def _workspace(self, d: int, dtype=torch.float32):
        lib = _lib.load()
        # plan preparation, once per matrix: a bf16 product of 256 columns or more takes the hub pass in its wide layout
        if dtype == torch.bfloat16 and d >= 256 and not getattr(self, "_wide_tried", False) and self.n_hub_rows > 0:
            self.build_hub_wide()
        query = lib.plx_spmm_workspace_bytes_bf16 if dtype == torch.bfloat16 else lib.plx_spmm_workspace_bytes
        need = int(query(self._plan, d))
        if need == 0:
            return None, 0
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device=self.device)
        return self._ws, need

    def to_torch(self) -> torch.Tensor:
        return torch.sparse_csr_tensor(
            self.rowptr.to(torch.int64), self.col.to(torch.int64), self.val, size=self.shape, device=self.device
        )


def _aligned_workspace(nbytes: int, device) -> torch.Tensor:
    """uint8 scratch whose data pointer is 256-byte aligned (torch's allocator hands out 512-byte aligned blocks)."""
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
    assert ws.data_ptr() % 256 == 0
    return ws


def csr_transpose(a: CsrMatrix, seg_len: int = 0) -> CsrMatrix:
    """The CSR of A^T, built on the device (what the reference's loader builds on the host, dataloader.py:368)."""
    m, k = a.shape
    lib = _lib.load()
    rowptr_t = torch.empty(k + 1, dtype=torch.int32, device=a.device)
    col_t = torch.empty(a.nnz, dtype=torch.int32, device=a.device)
    val_t = torch.empty(a.nnz, dtype=torch.float32, device=a.device)
    need = int(lib.plx_csr_transpose_workspace_bytes(m, k, a.nnz))
    ws = _aligned_workspace(need, a.device)
    check(
        lib.plx_csr_transpose_f32(m, k, a.nnz, a.rowptr.data_ptr(), a.col.data_ptr() if a.nnz else None,
                                  a.val.data_ptr() if a.nnz else None, rowptr_t.data_ptr(), col_t.data_ptr() if a.nnz else None,
                                  val_t.data_ptr() if a.nnz else None, ws.data_ptr(), need, _stream()),
        "plx_csr_transpose_f32",
    )
    return CsrMatrix(rowptr_t, col_t, val_t, (k, m), seg_len, defer_plan=True)


def csr_pair_from_edges(edge_index: torch.Tensor, edge_weight: torch.Tensor, shape, row_range=None, col_range=None,
                        seg_len: int = 0):
    """(A, A^T) of a rank's block from an edge list, on the device.

    Counterpart of the loader's ``__split_adj`` (plexus/utils/dataloader.py:327-375): mask the edges to
    ``row_range x col_range``, re-base, build the CSR (duplicates summed) and the CSR of its transpose."""
    a = csr_from_edges(edge_index, edge_weight, shape, row_range, col_range, seg_len)
    return a, csr_transpose(a, seg_len)


def csr_from_edges(edge_index: torch.Tensor, edge_weight: torch.Tensor, shape, row_range=None, col_range=None,
                   seg_len: int = 0) -> "CsrMatrix":
    """The CSR block ``row_range x col_range`` of an edge list (plexus/utils/dataloader.py:343-367): edges outside
    the block are dropped, the rest re-based, sorted by (row, column) and duplicates summed."""
    _need_gpu(edge_index, edge_weight)
    r0, r1 = row_range if row_range is not None else (0, int(shape[0]))
    c0, c1 = col_range if col_range is not None else (0, int(shape[1]))
    ei = edge_index.to(torch.int64)
    rows, cols = ei[0].contiguous(), ei[1].contiguous()
    w = edge_weight.to(torch.float32).contiguous()
    n = int(rows.numel())
    lib = _lib.load()
    mb, kb = r1 - r0, c1 - c0
    rowptr = torch.empty(mb + 1, dtype=torch.int32, device=w.device)
    col_out = torch.empty(max(n, 1), dtype=torch.int32, device=w.device)
    val_out = torch.empty(max(n, 1), dtype=torch.float32, device=w.device)
    need = int(lib.plx_coo_block_to_csr_workspace_bytes(n, mb, kb))
    ws = _aligned_workspace(need, w.device)
    nnz = _lib.C.c_int64(0)
    check(
        lib.plx_coo_block_to_csr_f32(n, rows.data_ptr() if n else None, cols.data_ptr() if n else None, w.data_ptr() if n else None,
                                     r0, r1, c0, c1, rowptr.data_ptr(), col_out.data_ptr(), val_out.data_ptr(), _lib.C.byref(nnz),
                                     ws.data_ptr(), need, _stream()),
        "plx_coo_block_to_csr_f32",
    )
    del ws
    k = int(nnz.value)
    return CsrMatrix(rowptr, _trimmed(col_out, k), _trimmed(val_out, k), (mb, kb), seg_len, defer_plan=True)


def _trimmed(t: torch.Tensor, k: int) -> torch.Tensor:
    """The first k entries of a buffer sized for the worst case: a view when little is wasted, else a copy."""
    return t[:k] if k * 10 >= t.numel() * 9 else t[:k].clone()


def gcn_norm_from_edges(edge_index: torch.Tensor, edge_weight: Optional[torch.Tensor], num_nodes: int,
                        transposed: bool = False, seg_len: int = 0) -> "CsrMatrix":
    """D^-1/2 (A + I) D^-1/2 (its transpose with ``transposed``) as a CSR matrix from an edge list, in one call:
    missing self loops get weight 1, d is the weighted in-degree, duplicate edges are summed -- T.GCNNorm and the
    CSR conversion of plexus/utils/dataset.py:101,158-168."""
    _need_gpu(edge_index)
    ei = edge_index.to(torch.int64)
    rows, cols = ei[0].contiguous(), ei[1].contiguous()
    w = None if edge_weight is None else edge_weight.to(torch.float32).contiguous()
    n_edges, n = int(rows.numel()), int(num_nodes)
    lib = _lib.load()
    dev = edge_index.device
    rowptr = torch.empty(n + 1, dtype=torch.int32, device=dev)
    col_out = torch.empty(max(n_edges + n, 1), dtype=torch.int32, device=dev)
    val_out = torch.empty(max(n_edges + n, 1), dtype=torch.float32, device=dev)
    need = int(lib.plx_gcn_norm_edges_workspace_bytes(n_edges, n))
    ws = _aligned_workspace(need, dev)
    nnz = _lib.C.c_int64(0)
    check(
        lib.plx_gcn_norm_edges_f32(n_edges, rows.data_ptr() if n_edges else None, cols.data_ptr() if n_edges else None,
                                   w.data_ptr() if (w is not None and n_edges) else None, n, int(bool(transposed)),
                                   rowptr.data_ptr(), col_out.data_ptr(), val_out.data_ptr(), _lib.C.byref(nnz), ws.data_ptr(), need,
                                   _stream()),
        "plx_gcn_norm_edges_f32",
    )
    del ws
    k = int(nnz.value)
    return CsrMatrix(rowptr, _trimmed(col_out, k), _trimmed(val_out, k), (n, n), seg_len, defer_plan=True)


def csr_permute(a: "CsrMatrix", perm_rows: torch.Tensor, perm_cols: torch.Tensor, a_t: Optional["CsrMatrix"] = None,
                seg_len: int = 0) -> "CsrMatrix":
    """P_rows . A . P_cols^T with P[i, perm[i]] = 1 as a CSR matrix: entry (i, j) of the result is entry
    (perm_rows[i], perm_cols[j]) of A (plexus/utils/dataset.py:137-190).

    Works from the CSR of A^T (``a_t``; built here when not given -- pass it when several permutations of one
    matrix are wanted): its rows are walked in the order perm_cols, the row ids in them renumbered, and one stable
    sort by the new row id leaves every row of the result in ascending column order."""
    a = as_csr(a)
    _need_gpu(perm_rows, perm_cols)
    m, k = a.shape
    if perm_rows.numel() != m or perm_cols.numel() != k:
        raise ValueError("csr_permute: a %dx%d matrix needs permutations of %d rows and %d columns" % (m, k, m, k))
    if a_t is None:
        a_t = csr_transpose(a)
    elif a_t.shape != (k, m) or a_t.nnz != a.nnz:
        raise ValueError("csr_permute: a_t is not the transpose of a")
    walk = perm_cols.to(torch.int64).contiguous()
    new_row = invert_permutation(perm_rows)
    lib = _lib.load()
    rowptr = torch.empty(m + 1, dtype=torch.int32, device=a.device)
    col_out = torch.empty(a.nnz, dtype=torch.int32, device=a.device)
    val_out = torch.empty(a.nnz, dtype=torch.float32, device=a.device)
    need = int(lib.plx_csr_permute_transposed_workspace_bytes(k, m, a.nnz))
    ws = _aligned_workspace(need, a.device)
    check(
        lib.plx_csr_permute_transposed_f32(k, m, a.nnz, a_t.rowptr.data_ptr(), a_t.col.data_ptr() if a.nnz else None,
                                           a_t.val.data_ptr() if a.nnz else None, walk.data_ptr() if k else None,
                                           new_row.data_ptr() if m else None, rowptr.data_ptr(), col_out.data_ptr() if a.nnz else None,
                                           val_out.data_ptr() if a.nnz else None, ws.data_ptr(), need, _stream()),
        "plx_csr_permute_transposed_f32",
    )
    return CsrMatrix(rowptr, col_out, val_out, (m, k), seg_len, defer_plan=True)


def invert_permutation(perm: torch.Tensor) -> torch.Tensor:
    """inv with inv[perm[i]] = i (int64, on the device)."""
    _need_gpu(perm)
    perm = perm.to(torch.int64).contiguous()
    inv = torch.full_like(perm, -1)  # a slot no entry of perm names stays -1, which the users of the map refuse
    check(_lib.load().plx_invert_permutation_i64(perm.numel(), perm.data_ptr(), inv.data_ptr(), _stream()), "plx_invert_permutation_i64")
    return inv


def relabel_edges(edge_index: torch.Tensor, map_row: torch.Tensor, map_col: torch.Tensor) -> torch.Tensor:
    """Edge list with (row, col) replaced by (map_row[row], map_col[col]) -- the vertex relabelling that the
    reference writes as P.A.P2^T (plexus/utils/dataset.py:137-190) when the maps are the inverse permutations."""
    _need_gpu(edge_index, map_row, map_col)
    ei = edge_index.to(torch.int64).contiguous()
    map_row = map_row.to(torch.int64).contiguous()
    map_col = map_col.to(torch.int64).contiguous()
    out = torch.empty_like(ei)
    n = int(ei.shape[1])
    check(
        _lib.load().plx_relabel_edges_i64(n, ei[0].data_ptr(), ei[1].data_ptr(), map_row.data_ptr(), map_row.numel(),
                                          map_col.data_ptr(), map_col.numel(), out[0].data_ptr(), out[1].data_ptr(), _stream()),
        "plx_relabel_edges_i64",
    )
    return out


def csr_to_edges(a: "CsrMatrix"):
    """(edge_index int64 [2, nnz], edge_weight) of a CSR matrix in storage order (rows, then columns, ascending),
    as to_edge_index gives them in plexus/utils/dataset.py:195-216."""
    a = as_csr(a)
    nnz = int(a.col.numel())
    ei = torch.empty((2, nnz), dtype=torch.int64, device=a.col.device)
    check(
        _lib.load().plx_csr_to_coo_i64(a.shape[0], nnz, a.rowptr.data_ptr(), a.col.data_ptr() if nnz else None,
                                       ei[0].data_ptr() if nnz else None, ei[1].data_ptr() if nnz else None, _stream()),
        "plx_csr_to_coo_i64",
    )
    return ei, a.val


def as_csr(a, seg_len: int = 0) -> CsrMatrix:
    """CsrMatrix of ``a``; a torch CSR tensor is converted once and the result is cached on it."""
    if isinstance(a, CsrMatrix):
        return a
    cached = getattr(a, "_plexus_amd_csr", None)
    if cached is None:
        cached = CsrMatrix.from_torch(a, seg_len)
        try:
            a._plexus_amd_csr = cached
        except Exception:
            pass
    return cached


def spmm(a, h: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Y = A.H (fp32 or bf16 H; fp32 accumulation)."""
    a = as_csr(a)
    _need_gpu(h)
    h = _rowmajor(h)
    m, k = a.shape
    if h.shape[0] != k:
        raise ValueError("spmm: A is %dx%d but H has %d rows" % (m, k, h.shape[0]))
    d = h.shape[1]
    if out is None:
        out = torch.empty((m, d), dtype=h.dtype, device=h.device)
    ws, ws_bytes = a._workspace(d, h.dtype)
    lib = _lib.load()
    fn = {torch.float32: lib.plx_spmm_csr_f32, torch.bfloat16: lib.plx_spmm_csr_bf16}.get(h.dtype)
    if fn is None:
        raise TypeError("spmm: unsupported dtype %s" % h.dtype)
    if out.dtype != h.dtype:
        raise TypeError("spmm: out dtype differs from H")
    check(
        fn(a._plan, a.val.data_ptr(), h.data_ptr(), _ld(h), d, out.data_ptr(), _ld(out),
           ws.data_ptr() if ws is not None else None, ws_bytes, _stream()),
        "plx_spmm_csr",
    )
    return out


def chunked_spmm(a, h: torch.Tensor, max_rows_per_chunk: int = 1000000, on_chunk=None) -> torch.Tensor:
    """Row-chunked Y = A.H with the reference's chunk boundaries (plexus/gcn_conv.py:77-91).

    Each chunk is one launch writing its rows of the full output (the hub pass of a plan that has one runs with the first
    chunk, for all of them); ``on_chunk(i, (start, end), y)`` is called after chunk i has been enqueued (the place where
    the reference starts the chunk's all-reduce, gcn_conv.py:103-110).  The rows are bit-identical to the un-chunked product."""
    a = as_csr(a)
    _need_gpu(h)
    h = _rowmajor(h)
    lib = _lib.load()
    fn = {torch.float32: lib.plx_spmm_csr_chunk_f32, torch.bfloat16: lib.plx_spmm_csr_chunk_bf16}.get(h.dtype)
    if fn is None:
        raise TypeError("chunked_spmm: unsupported dtype %s" % h.dtype)
    m, k = a.shape
    if h.shape[0] != k:
        raise ValueError("chunked_spmm: A is %dx%d but H has %d rows" % (m, k, h.shape[0]))
    d = h.shape[1]
    y = torch.empty((m, d), dtype=h.dtype, device=h.device)
    ws, ws_bytes = a._workspace(d, h.dtype)
    num_chunks = max(1, (m + max_rows_per_chunk - 1) // max_rows_per_chunk)
    rows_per_chunk = m // num_chunks
    for i in range(num_chunks):
        start = i * rows_per_chunk
        end = m if i == num_chunks - 1 else (i + 1) * rows_per_chunk
        check(
            fn(a._plan, start, end, int(i == 0), a.val.data_ptr(), h.data_ptr(), _ld(h), d, y.data_ptr(), _ld(y),
               ws.data_ptr() if ws is not None else None, ws_bytes, _stream()),
            "plx_spmm_csr_chunk",
        )
        if on_chunk is not None:
            on_chunk(i, (start, end), y)
    return y


# fp32 products run on the bf16 matrix cores from exact three-way splits of the operands (fp32-level accuracy)
# when the operands are aligned for it; PLEXUS_FP32_GEMM=mfma32 keeps every product on the fp32 MFMA kernels.
SPLIT_GEMM = os.environ.get("PLEXUS_FP32_GEMM", "split") != "mfma32"


def _split_ok(n: int, k: int, *mats) -> bool:
    if not SPLIT_GEMM or k <= 0:
        return False
    if n <= 128 and k <= 128:  # the kernel for small weights takes any alignment
        return True
    return k % 2 == 0 and all(t is None or (t.data_ptr() % 8 == 0 and _ld(t) % 2 == 0) for t in mats)


def _split_ws(n: int, k: int, device):
    need = int(_lib.load().plx_gemm_f32_split_workspace_bytes(n, k))
    return _aligned_workspace(need, device), need


def _new_bits(m: int, n: int, device) -> torch.Tensor:
    """int32 [m x ceil(n / 32)] with rows of a multiple of four words (the products read a row's bits with one 128-bit load)."""
    words = (n + 31) // 32
    return torch.empty((m, (words + 3) // 4 * 4), dtype=torch.int32, device=device)[:, :words]


def sign_bits(x: torch.Tensor) -> torch.Tensor:
    """One bit per element of an fp32 matrix: bit c % 32 of word [row, c // 32] is set when x[row, c] > 0 (int32 words)."""
    _need_gpu(x)
    _need_fp32("sign_bits", x=x)
    x = _rowmajor(x)
    m, n = x.shape
    bits = _new_bits(m, n, x.device)
    check(_lib.load().plx_sign_bits_f32(m, n, x.data_ptr(), _ld(x), bits.data_ptr(), _ld(bits), _stream()), "plx_sign_bits_f32")
    return bits


def dropout_(x: torch.Tensor, p: float, seed: int = 0, offset: int = 0) -> torch.Tensor:
    """In-place dropout of an fp32 matrix with the counter-based mask of the fused products (kept elements scaled by
    1 / (1 - p)); the form the products use for operands their kernels do not take."""
    _need_gpu(x)
    _need_fp32("dropout_", x=x)
    if x.dim() != 2 or (x.shape[1] > 1 and x.stride(1) != 1):
        raise ValueError("dropout_: a 2-D tensor with contiguous rows is expected")
    check(_lib.load().plx_dropout_f32(x.shape[0], x.shape[1], x.data_ptr(), _ld(x), float(p), int(seed), int(offset), _stream()),
          "plx_dropout_f32")
    return x


def gemm_nn(a: torch.Tensor, b: torch.Tensor, relu: bool = False, out: Optional[torch.Tensor] = None, want_bits: bool = False,
            dropout_p: float = 0.0, seed: int = 0, offset: int = 0):
    """C = A.B, optionally max(C, 0), optionally dropout after that (the mask of ``gemm_nt_bf16``); ``out`` may be a column
    slice of a wider matrix.  With ``want_bits`` the result is (C, sign bits of C as by ``sign_bits``): the mask of the
    layer (ReLU and dropout) in the form ``gemm_nt(mask_bits=)`` reads."""
    _need_gpu(a, b, out)
    _need_fp32("gemm_nn", a=a, b=b)
    a, b = _rowmajor(a), _rowmajor(b)
    m, k = a.shape
    k2, n = b.shape
    if k != k2:
        raise ValueError("gemm_nn: inner dimensions differ (%d vs %d)" % (k, k2))
    if out is None:
        c = torch.empty((m, n), dtype=torch.float32, device=a.device)
    else:
        c = out
        if tuple(c.shape) != (m, n) or c.dtype != torch.float32 or (n > 1 and c.stride(1) != 1):
            raise ValueError("gemm_nn: out must be fp32 [%d x %d] with contiguous rows" % (m, n))
    if dropout_p > 0.0:
        bits = _new_bits(m, n, a.device) if want_bits else None
        if _split_ok(n, k, a):
            ws, need = _split_ws(n, k, a.device)
            check(
                _lib.load().plx_gemm_nn_f32_split_dropout(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                                          (PLX_GEMM_RELU if relu else 0) | PLX_GEMM_DROPOUT, float(dropout_p), int(seed),
                                                          int(offset), bits.data_ptr() if want_bits else None,
                                                          _ld(bits) if want_bits else 0, ws.data_ptr(), need, _stream()),
                "plx_gemm_nn_f32_split_dropout",
            )
            return (c, bits) if want_bits else c
        check(
            _lib.load().plx_gemm_nn_f32(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                        PLX_GEMM_RELU if relu else 0, _stream()),
            "plx_gemm_nn_f32",
        )
        dropout_(c, dropout_p, seed, offset)
        return (c, sign_bits(c)) if want_bits else c
    if _split_ok(n, k, a):
        ws, need = _split_ws(n, k, a.device)
        if want_bits:
            bits = _new_bits(m, n, a.device)
            check(
                _lib.load().plx_gemm_nn_f32_split_bits(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                                       PLX_GEMM_RELU if relu else 0, bits.data_ptr(), _ld(bits), ws.data_ptr(),
                                                       need, _stream()),
                "plx_gemm_nn_f32_split_bits",
            )
            return c, bits
        check(
            _lib.load().plx_gemm_nn_f32_split(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                              PLX_GEMM_RELU if relu else 0, ws.data_ptr(), need, _stream()),
            "plx_gemm_nn_f32_split",
        )
        return c
    check(
        _lib.load().plx_gemm_nn_f32(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                    PLX_GEMM_RELU if relu else 0, _stream()),
        "plx_gemm_nn_f32",
    )
    return (c, sign_bits(c)) if want_bits else c


def _device_scalar(value: float, device) -> torch.Tensor:
    return torch.full((1,), float(value), dtype=torch.float32, device=device)


def gemm_nt(a: torch.Tensor, b: torch.Tensor, mask: Optional[torch.Tensor] = None,
            mask_bits: Optional[torch.Tensor] = None, alpha: float = 1.0) -> torch.Tensor:
    """C = alpha * (A * [mask > 0]).B^T with B stored [N x K].  ``mask_bits`` (``sign_bits(mask)``, or the second result of
    ``gemm_nn(want_bits=True)``) lets the product read the mask as one bit per element where its kernel can."""
    _need_gpu(a, b, mask)
    _need_fp32("gemm_nt", a=a, b=b, mask=mask)
    a, b = _rowmajor(a), _rowmajor(b)
    m, k = a.shape
    n, k2 = b.shape
    if k != k2:
        raise ValueError("gemm_nt: inner dimensions differ (%d vs %d)" % (k, k2))
    if mask is not None:
        mask = _rowmajor(mask)
        if mask.shape != a.shape:
            raise ValueError("gemm_nt: mask shape differs from A")
    c = torch.empty((m, n), dtype=torch.float32, device=a.device)
    if mask_bits is not None:
        if mask is None or mask_bits.dtype != torch.int32 or mask_bits.dim() != 2 or mask_bits.shape[0] != m or \
                mask_bits.shape[1] < (k + 31) // 32 or mask_bits.stride(1) != 1:
            raise ValueError("gemm_nt: mask_bits must be int32 [%d x >= %d] beside the fp32 mask" % (m, (k + 31) // 32))
    if _split_ok(n, k, a, mask) and alpha != 1.0:
        ws, need = _split_ws(n, k, a.device)
        check(
            _lib.load().plx_gemm_nt_f32_split_scaled(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                                     mask.data_ptr() if mask is not None else None,
                                                     _ld(mask) if mask is not None else 0,
                                                     mask_bits.data_ptr() if mask_bits is not None else None,
                                                     _ld(mask_bits) if mask_bits is not None else 0, float(alpha),
                                                     ws.data_ptr(), need, _stream()),
            "plx_gemm_nt_f32_split_scaled",
        )
        return c
    if _split_ok(n, k, a, mask):
        ws, need = _split_ws(n, k, a.device)
        if mask_bits is not None:
            check(
                _lib.load().plx_gemm_nt_f32_split_bits(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                                       mask.data_ptr(), _ld(mask), mask_bits.data_ptr(), _ld(mask_bits),
                                                       ws.data_ptr(), need, _stream()),
                "plx_gemm_nt_f32_split_bits",
            )
            return c
        check(
            _lib.load().plx_gemm_nt_f32_split(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                              mask.data_ptr() if mask is not None else None,
                                              _ld(mask) if mask is not None else 0, ws.data_ptr(), need, _stream()),
            "plx_gemm_nt_f32_split",
        )
        return c
    check(
        _lib.load().plx_gemm_nt_f32(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                    mask.data_ptr() if mask is not None else None,
                                    _ld(mask) if mask is not None else 0, _stream()),
        "plx_gemm_nt_f32",
    )
    return c if alpha == 1.0 else scale_by_scalar(c, _device_scalar(alpha, c.device))  # operands the split kernels do not take


def gemm_tn(a: torch.Tensor, b: torch.Tensor, mask: Optional[torch.Tensor] = None, alpha: float = 1.0,
            mask_bits: Optional[torch.Tensor] = None) -> torch.Tensor:
    """C[K x N] = alpha * A[M x K]^T.(B * [mask > 0])[M x N].  ``mask_bits`` (``sign_bits(mask)``) lets the product read
    the mask as one bit per element."""
    _need_gpu(a, b, mask)
    _need_fp32("gemm_tn", a=a, b=b, mask=mask)
    a, b = _rowmajor(a), _rowmajor(b)
    m, k = a.shape
    m2, n = b.shape
    if m != m2:
        raise ValueError("gemm_tn: row counts differ (%d vs %d)" % (m, m2))
    if mask is not None:
        mask = _rowmajor(mask)
        if mask.shape != b.shape:
            raise ValueError("gemm_tn: mask shape differs from B")
    lib = _lib.load()
    c = torch.empty((k, n), dtype=torch.float32, device=a.device)
    if mask_bits is not None:
        if mask is None or mask_bits.dtype != torch.int32 or mask_bits.dim() != 2 or mask_bits.shape[0] != m or \
                mask_bits.shape[1] < (n + 31) // 32 or mask_bits.stride(1) != 1:
            raise ValueError("gemm_tn: mask_bits must be int32 [%d x >= %d] beside the fp32 mask" % (m, (n + 31) // 32))
    if SPLIT_GEMM and k > 0 and n > 0:
        need = int(lib.plx_gemm_tn_f32_split_workspace_bytes(m, n, k))
        ws = _aligned_workspace(need, a.device)
        check(
            lib.plx_gemm_tn_f32_split(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                      mask.data_ptr() if mask is not None else None, _ld(mask) if mask is not None else 0,
                                      mask_bits.data_ptr() if mask_bits is not None else None,
                                      _ld(mask_bits) if mask_bits is not None else 0, float(alpha), ws.data_ptr(), need, _stream()),
            "plx_gemm_tn_f32_split",
        )
        return c
    need = int(lib.plx_gemm_tn_workspace_bytes(m, n, k))
    ws = torch.empty(need, dtype=torch.uint8, device=a.device) if need else None
    check(
        lib.plx_gemm_tn_f32(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                            mask.data_ptr() if mask is not None else None, _ld(mask) if mask is not None else 0,
                            ws.data_ptr() if ws is not None else None, need, _stream()),
        "plx_gemm_tn_f32",
    )
    return c if alpha == 1.0 else scale_by_scalar(c, _device_scalar(alpha, c.device))  # K x N elements: a weight's worth


def cast_bf16(x: torch.Tensor, transpose: bool = False) -> torch.Tensor:
    """bf16(x) or bf16(x^T) of an fp32 matrix."""
    _need_gpu(x)
    x = _rowmajor(x)
    if x.dtype != torch.float32:
        raise TypeError("cast_bf16: fp32 input expected")
    m, n = x.shape
    y = torch.empty((n, m) if transpose else (m, n), dtype=torch.bfloat16, device=x.device)
    check(_lib.load().plx_cast_f32_bf16(m, n, x.data_ptr(), _ld(x), y.data_ptr(), _ld(y), int(transpose), _stream()),
          "plx_cast_f32_bf16")
    return y


def bf16_bits_supported(n: int, k: int) -> bool:
    """Whether ``gemm_nt_bf16(want_bits=True)`` can write the sign bits of an M x n result of a k-wide contraction."""
    return 0 < n <= 256 and 8 <= k <= 256 and n % 8 == 0 and k % 8 == 0


def gemm_nt_bf16(a: torch.Tensor, b: torch.Tensor, mask: Optional[torch.Tensor] = None, alpha: float = 1.0,
                 relu: bool = False, dropout_p: float = 0.0, seed: int = 0, offset: int = 0,
                 mask_bits: Optional[torch.Tensor] = None, want_bits: bool = False):
    """bf16 C = epilogue(alpha * (A * [mask > 0]) . B^T), B stored [N x K]; optional ReLU then dropout.

    ``mask_bits``: the same mask as one bit per element (int32 words, as ``want_bits`` returns them), read in its place
    where the kernel can.  With ``want_bits`` the result is (C, bits): bit c % 32 of word [r, c // 32] says that C[r, c]
    is positive (``bf16_bits_supported`` tells for which shapes)."""
    _need_gpu(a, b, mask)
    a, b = _rowmajor(a), _rowmajor(b)
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise TypeError("gemm_nt_bf16: bf16 operands expected")
    m, k = a.shape
    n, k2 = b.shape
    if k != k2:
        raise ValueError("gemm_nt_bf16: inner dimensions differ (%d vs %d)" % (k, k2))
    if mask is not None:
        mask = _rowmajor(mask)
        if mask.shape != a.shape or mask.dtype != torch.bfloat16:
            raise ValueError("gemm_nt_bf16: mask must be bf16 with the shape of A")
    if mask_bits is not None:
        _need_gpu(mask_bits)
        if mask is None or mask_bits.dtype != torch.int32 or mask_bits.dim() != 2 or mask_bits.shape[0] != m \
                or mask_bits.stride(1) != 1 or mask_bits.shape[1] * 32 < k:
            raise ValueError("gemm_nt_bf16: mask_bits must be int32 words [M, >= ceil(K / 32)] beside the bf16 mask")
    c = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    bits = _new_bits(m, n, a.device) if want_bits else None
    flags = (PLX_GEMM_RELU if relu else 0) | (PLX_GEMM_DROPOUT if dropout_p > 0.0 else 0)
    check(
        _lib.load().plx_gemm_nt_bf16_bits(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                          mask.data_ptr() if mask is not None else None, _ld(mask) if mask is not None else 0,
                                          mask_bits.data_ptr() if mask_bits is not None else None,
                                          _ld(mask_bits) if mask_bits is not None else 0,
                                          bits.data_ptr() if bits is not None else None, _ld(bits) if bits is not None else 0,
                                          float(alpha), flags, float(dropout_p), int(seed), int(offset), _stream()),
        "plx_gemm_nt_bf16_bits",
    )
    return (c, bits) if want_bits else c


def gemm_tn_bf16(a: torch.Tensor, b: torch.Tensor, mask: Optional[torch.Tensor] = None, alpha: float = 1.0,
                 mask_bits: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 C[K x N] = alpha * A[M x K]^T . (B * [mask > 0])[M x N] from bf16 operands; ``mask_bits``: the mask as one
    bit per element (int32 words [M, >= ceil(N / 32)]), read in its place where the kernel can."""
    _need_gpu(a, b, mask)
    a, b = _rowmajor(a), _rowmajor(b)
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise TypeError("gemm_tn_bf16: bf16 operands expected")
    m, k = a.shape
    m2, n = b.shape
    if m != m2:
        raise ValueError("gemm_tn_bf16: row counts differ (%d vs %d)" % (m, m2))
    if mask is not None:
        mask = _rowmajor(mask)
        if mask.shape != b.shape or mask.dtype != torch.bfloat16:
            raise ValueError("gemm_tn_bf16: mask must be bf16 with the shape of B")
    if mask_bits is not None:
        _need_gpu(mask_bits)
        if mask is None or mask_bits.dtype != torch.int32 or mask_bits.dim() != 2 or mask_bits.shape[0] != m \
                or mask_bits.stride(1) != 1 or mask_bits.shape[1] * 32 < n:
            raise ValueError("gemm_tn_bf16: mask_bits must be int32 words [M, >= ceil(N / 32)] beside the bf16 mask")
    lib = _lib.load()
    c = torch.empty((k, n), dtype=torch.float32, device=a.device)
    need = int(lib.plx_gemm_tn_bf16_workspace_bytes(m, n, k))
    ws = torch.empty(need, dtype=torch.uint8, device=a.device) if need else None
    check(
        lib.plx_gemm_tn_bf16_bits(m, n, k, a.data_ptr(), _ld(a), b.data_ptr(), _ld(b), c.data_ptr(), _ld(c),
                                  mask.data_ptr() if mask is not None else None, _ld(mask) if mask is not None else 0,
                                  mask_bits.data_ptr() if mask_bits is not None else None,
                                  _ld(mask_bits) if mask_bits is not None else 0,
                                  float(alpha), ws.data_ptr() if ws is not None else None, need, _stream()),
        "plx_gemm_tn_bf16_bits",
    )
    return c


def copy_rows(src: torch.Tensor, dst: torch.Tensor) -> torch.Tensor:
    """dst[:, :] = src for two row-major matrices of one shape and dtype with any row pitches (no torch kernel)."""
    _need_gpu(src, dst)
    if src.shape != dst.shape or src.dtype != dst.dtype or src.dim() != 2:
        raise ValueError("copy_rows: two 2-D tensors of one shape and dtype expected")
    src = _rowmajor(src)
    if dst.shape[1] > 1 and dst.stride(1) != 1:
        raise ValueError("copy_rows: the rows of the destination must be contiguous")
    es = src.element_size()
    m, n = src.shape
    check(_lib.load().plx_copy_rows(m, n * es, src.data_ptr(), _ld(src) * es, dst.data_ptr(), _ld(dst) * es, _stream()), "plx_copy_rows")
    return dst


def relu(x: torch.Tensor, inplace: bool = False) -> torch.Tensor:
    _need_gpu(x)
    if x.dtype != torch.float32 or x.dim() != 2:
        raise TypeError("relu: a 2-D fp32 tensor is expected (bf16 layers fuse the ReLU into the product)")
    if not inplace:
        x = _rowmajor(x)
    y = x if inplace else torch.empty(x.shape, dtype=torch.float32, device=x.device)
    check(_lib.load().plx_relu_f32(x.shape[0], x.shape[1], x.data_ptr(), _ld(x), y.data_ptr(), _ld(y), _stream()), "plx_relu_f32")
    return y


def relu_bwd(dy: torch.Tensor, y: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _need_gpu(dy, y, out)
    if dy.dtype != torch.float32 or y.dtype != torch.float32 or dy.shape != y.shape:
        raise TypeError("relu_bwd: two fp32 tensors of one shape are expected")
    dy, y = _rowmajor(dy), _rowmajor(y)
    dx = out if out is not None else torch.empty(dy.shape, dtype=torch.float32, device=dy.device)
    check(
        _lib.load().plx_relu_bwd_f32(dy.shape[0], dy.shape[1], dy.data_ptr(), _ld(dy), y.data_ptr(), _ld(y),
                                     dx.data_ptr(), _ld(dx), _stream()),
        "plx_relu_bwd_f32",
    )
    return dx


def softmax_xent(logits: torch.Tensor, labels: torch.Tensor, num_nodes: int, num_classes: int, row_offset: int = 0,
                 gscale: float = 1.0, want_grad: bool = True):
    """(loss[1], dlogits or None) of the masked row-softmax cross-entropy."""
    _need_gpu(logits, labels)
    logits = _rowmajor(logits)
    if labels.dtype != torch.int64:
        labels = labels.to(torch.int64)
    labels = labels.contiguous()
    m, c = logits.shape
    if labels.numel() != m:
        raise ValueError("softmax_xent: %d labels for %d rows" % (labels.numel(), m))
    lib = _lib.load()
    fn = {torch.float32: lib.plx_softmax_xent_f32, torch.bfloat16: lib.plx_softmax_xent_bf16}.get(logits.dtype)
    if fn is None:
        raise TypeError("softmax_xent: unsupported dtype %s" % logits.dtype)
    loss = torch.empty(1, dtype=torch.float32, device=logits.device)
    dlogits = None
    if want_grad:
        # the gradient takes the row pitch of the logits: a consumer that padded its rows (for 16-byte loads) gets it
        # back in the same layout
        ld = _ld(logits)
        dlogits = torch.empty((m, ld), dtype=logits.dtype, device=logits.device)[:, :c] if ld != c else \
            torch.empty((m, c), dtype=logits.dtype, device=logits.device)
    need = int(lib.plx_softmax_xent_workspace_bytes(m, c))
    ws = torch.empty(need, dtype=torch.uint8, device=logits.device)
    check(
        fn(m, c, logits.data_ptr(), _ld(logits), labels.data_ptr(), int(num_nodes),
                                 int(num_classes), int(row_offset), float(gscale), loss.data_ptr(),
                                 dlogits.data_ptr() if want_grad else None, _ld(dlogits) if want_grad else c,
                                 ws.data_ptr(), need, _stream()),
        "plx_softmax_xent",
    )
    return loss, dlogits


def _whole_padded_rows(x: torch.Tensor):
    """The [rows x pitch] matrix behind a row-major 2-D view whose rows are padded, if the view starts its storage and the
    storage holds every padded row whole; else None."""
    if x.dim() != 2 or x.shape[0] == 0 or x.shape[1] == 0 or x.stride(1) != 1 or x.stride(0) <= x.shape[1] or x.storage_offset() != 0:
        return None
    m, ld = x.shape[0], x.stride(0)
    if x.untyped_storage().nbytes() < m * ld * x.element_size():
        return None
    return x.as_strided((m, ld), (ld, 1))


def scale_by_scalar(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """x * scale for a one-element fp32 device tensor ``scale`` (read on the device; the host does not wait for it)."""
    _need_gpu(x, scale)
    if scale.numel() != 1:
        raise ValueError("scale_by_scalar: the scale must hold one element, got %d" % scale.numel())
    lib = _lib.load()
    fn = {torch.float32: lib.plx_scale_by_device_scalar_f32, torch.bfloat16: lib.plx_scale_by_device_scalar_bf16}.get(x.dtype)
    if fn is None:
        raise TypeError("scale_by_scalar: unsupported dtype %s" % x.dtype)
    scale = scale.detach().reshape(1).to(torch.float32)
    base = _whole_padded_rows(x)
    if base is not None:  # rows padded to a longer pitch, whole in their storage: scaled with their padding, layout kept
        yb = torch.empty_like(base)
        check(fn(base.numel(), base.data_ptr(), scale.data_ptr(), yb.data_ptr(), _stream()), "plx_scale_by_device_scalar")
        return yb[:, :x.shape[1]]
    x = x.contiguous()
    y = torch.empty_like(x)
    check(fn(x.numel(), x.data_ptr(), scale.data_ptr(), y.data_ptr(), _stream()), "plx_scale_by_device_scalar")
    return y


def gcn_norm_csr(a: CsrMatrix) -> torch.Tensor:
    """Values of D^-1/2 A D^-1/2 for a square CSR matrix that already holds its self loops."""
    if a.shape[0] != a.shape[1]:
        raise ValueError("gcn_norm_csr: square matrix required")
    out = torch.empty_like(a.val)
    dinv = torch.empty(a.shape[0], dtype=torch.float32, device=a.device)
    check(
        _lib.load().plx_gcn_norm_csr_f32(a.shape[0], a.rowptr.data_ptr(), a.col.data_ptr(), a.val.data_ptr(),
                                         out.data_ptr(), dinv.data_ptr(), _stream()),
        "plx_gcn_norm_csr_f32",
    )
    return out
