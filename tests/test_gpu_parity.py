"""Parity of the HIP path against the CPU oracle, through the C ABI, on the real GPU.

fp32 bar: max|x - ref| / max|ref| <= 1e-5 per output tensor; bf16 storage: <= 2e-2.
"""
import numpy as np
import pytest
import torch

from conftest import BF16_TOL, FP32_TOL, assert_parity, rel_err
from oracle import oracle_c
from oracle import plexus_oracle as po
from plexus_amd import ops
from plexus_amd.utils import synthetic as S

pytestmark = pytest.mark.gpu
DEV = "cuda"


def say(msg):
    print("[case] " + msg, flush=True)


def graph_small(kind="uniform", n=500, pairs=4000, seed=0, **kw):
    return S.build_graph(n, kind, 0, seed=seed, device="cpu", exact_pairs=pairs, **kw)


def to_dev(g, transpose=False, seg_len=0):
    if transpose:
        return ops.CsrMatrix(g.rowptr_t.to(DEV), g.col_t.to(DEV), g.val_t.to(DEV), (g.shape[1], g.shape[0]), seg_len)
    return ops.CsrMatrix(g.rowptr.to(DEV), g.col.to(DEV), g.val.to(DEV), g.shape, seg_len)


def oracle_spmm64(g, h, transpose=False):
    if transpose:
        return oracle_c.csr_spmm(g.rowptr_t.numpy(), g.col_t.numpy(), g.val_t.numpy(), h.numpy())
    return oracle_c.csr_spmm(g.rowptr.numpy(), g.col.numpy(), g.val.numpy(), h.numpy())


@pytest.mark.parametrize("d", [1, 2, 3, 4, 7, 16, 47, 64, 100, 128, 130, 256, 602, 1433, 2050])
def test_spmm_widths(d):
    say("spmm width D=%d" % d)
    g = graph_small(n=700, pairs=6000, seed=d)
    h = torch.randn(700, d, generator=torch.Generator().manual_seed(d))
    a = to_dev(g)
    y = ops.spmm(a, h.to(DEV)).cpu()
    ref_t = po.spmm(g.torch_csr(), h)  # the reference's operator on the host
    ref64 = oracle_spmm64(g, h)
    assert rel_err(y, ref64) <= FP32_TOL
    assert rel_err(y, ref_t) <= FP32_TOL


@pytest.mark.parametrize("seg_len", [4, 64, 1024])
@pytest.mark.parametrize("d", [8, 128, 602])
def test_spmm_power_law_with_split_rows(seg_len, d):
    say("spmm chung-lu seg_len=%d D=%d" % (seg_len, d))
    g = S.build_graph(3000, "chunglu", 40000, seed=1, device="cpu", gamma=2.1)
    assert g.degree_stats()["max_row_nnz"] > 1024
    h = torch.randn(3000, d, generator=torch.Generator().manual_seed(2))
    for transpose in (False, True):
        a = to_dev(g, transpose, seg_len)
        assert a.n_long_rows > 0 and a.n_segments >= 2 * a.n_long_rows
        y = ops.spmm(a, h.to(DEV)).cpu()
        assert rel_err(y, oracle_spmm64(g, h, transpose)) <= FP32_TOL


def test_spmm_edge_cases():
    say("spmm edge cases")
    # empty matrix rows, a matrix with no entries, a single hub row, rectangular block, padded ld
    m, k = 300, 200
    rowptr = torch.zeros(m + 1, dtype=torch.int64)
    col = torch.zeros(0, dtype=torch.int64)
    val = torch.zeros(0)
    a = ops.CsrMatrix(rowptr.to(DEV), col.to(DEV), val.to(DEV), (m, k))
    y = ops.spmm(a, torch.randn(k, 20, device=DEV))
    assert y.shape == (m, 20) and (y == 0).all()
    # hub: row 5 holds every column twice over the seg_len, all other rows empty
    gen = torch.Generator().manual_seed(0)
    counts = torch.zeros(m, dtype=torch.int64)
    counts[5] = k
    counts[299] = 3
    rowptr = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(counts, 0)])
    col = torch.cat([torch.arange(k), torch.tensor([0, 7, 199])])
    val = torch.rand(k + 3, generator=gen)
    h = torch.randn(k, 36, generator=gen)
    a = ops.CsrMatrix(rowptr.to(DEV), col.to(DEV), val.to(DEV), (m, k), seg_len=16)
    y = ops.spmm(a, h.to(DEV)).cpu()
    ref = oracle_c.csr_spmm(rowptr.numpy(), col.numpy(), val.numpy(), h.numpy())
    assert rel_err(y, ref) <= FP32_TOL
    assert (y[:5] == 0).all() and (y[6:299] == 0).all()
    # H and Y with a leading dimension larger than D (a column slab of a wider matrix)
    wide = torch.randn(k, 64, generator=gen)
    out_wide = torch.full((m, 80), 7.0, device=DEV)
    hd = wide.to(DEV)[:, 8:44]
    ops.spmm(a, hd, out=out_wide[:, 4:40])
    ref = oracle_c.csr_spmm(rowptr.numpy(), col.numpy(), val.numpy(), wide[:, 8:44].contiguous().numpy())
    assert rel_err(out_wide[:, 4:40].cpu(), ref) <= FP32_TOL
    assert (out_wide[:, :4] == 7).all() and (out_wide[:, 40:] == 7).all()
    # zero rows
    a0 = ops.CsrMatrix(torch.zeros(1, dtype=torch.int64, device=DEV), col[:0].to(DEV), val[:0].to(DEV), (0, k))
    assert ops.spmm(a0, h.to(DEV)).shape == (0, 36)


def test_spmm_plan_rejects_malformed_matrices():
    say("spmm plan: column out of range, decreasing rowptr, wrong nnz")
    from plexus_amd._lib import PlexusHipError

    rowptr = torch.tensor([0, 2, 3, 5], dtype=torch.int64)
    val = torch.ones(5)
    for bad_col in ([0, 1, 4, 2, 3], [0, -1, 2, 2, 3]):  # K = 4: columns 0..3 are valid
        with pytest.raises(PlexusHipError, match="column indices lie outside"):
            ops.CsrMatrix(rowptr.to(DEV), torch.tensor(bad_col).to(DEV), val.to(DEV), (3, 4))
    good_col = torch.tensor([0, 1, 3, 2, 3])
    with pytest.raises(PlexusHipError, match="rowptr decreases"):
        ops.CsrMatrix(torch.tensor([0, 3, 2, 5]).to(DEV), good_col.to(DEV), val.to(DEV), (3, 4))
    with pytest.raises(PlexusHipError, match="rowptr"):
        ops.CsrMatrix(torch.tensor([0, 2, 3, 4]).to(DEV), good_col.to(DEV), val.to(DEV), (3, 4))
    a = ops.CsrMatrix(rowptr.to(DEV), good_col.to(DEV), val.to(DEV), (3, 4))  # the well-formed one is accepted
    assert ops.spmm(a, torch.eye(4, device=DEV)).sum().item() == 5.0


def test_device_built_plan_tables_equal_the_host_construction():
    """The tables of the split rows are built on the device (compaction, prefix sum, one workgroup per split row); they
    must be exactly what the host routine makes of the same row pointers."""
    say("spmm plan tables: device against host")
    import ctypes as C

    from plexus_amd import _lib

    lib = _lib.load()
    gen = torch.Generator().manual_seed(0)
    for m, seg_len in ((5000, 7), (5000, 64), (1, 3), (300, 1), (70000, 16)):
        lens = torch.randint(0, 40, (m,), generator=gen)
        lens[torch.randint(0, m, (max(1, m // 50),), generator=gen)] = torch.randint(40, 3000, (max(1, m // 50),), generator=gen)
        rowptr = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(lens, 0)]).to(torch.int32)
        nnz = int(rowptr[-1])
        col = torch.zeros(nnz, dtype=torch.int32)
        a = ops.CsrMatrix(rowptr.to(DEV), col.to(DEV), torch.ones(nnz).to(DEV), (m, 4), seg_len)
        rp = rowptr.numpy()
        nl, ns = C.c_int64(), C.c_int64()
        assert lib.plx_spmm_segments_host(m, rp.ctypes.data, seg_len, C.byref(nl), C.byref(ns), None, None, 0, None, None, 0) == 0
        assert (a.n_long_rows, a.n_segments) == (nl.value, ns.value) and nl.value > 0
        want = [np.zeros(nl.value, np.int32), np.zeros(nl.value + 1, np.int32), np.zeros(ns.value, np.int32), np.zeros(ns.value, np.int32)]
        assert lib.plx_spmm_segments_host(m, rp.ctypes.data, seg_len, C.byref(nl), C.byref(ns), want[0].ctypes.data, want[1].ctypes.data,
                                          nl.value, want[2].ctypes.data, want[3].ctypes.data, ns.value) == 0
        got = [np.full_like(w, -1) for w in want]
        _lib.check(lib.plx_spmm_plan_tables_host(a._plan, *[x.ctypes.data for x in got]), "plx_spmm_plan_tables_host")
        for name, x, w in zip(("long_rows", "seg_first", "seg_begin", "seg_end"), got, want):
            assert np.array_equal(x, w), (name, m, seg_len)


def test_spmm_and_transpose_just_below_the_int32_limit():
    """Maximum size: 2,145,386,496 stored entries (the entry points take fewer than 2^31 - 64), every row split into two
    segments.  The product is checked against fp64 arithmetic by torch in row blocks, the transpose by the adjoint
    identity and by transposing twice."""
    say("spmm + transpose with 2.1e9 entries")
    m, per_row, band = 2 ** 21, 1023, 1024
    k, nnz, d = per_row * band, m * per_row, 4
    assert 2 ** 31 - 2 ** 21 <= nnz < 2 ** 31 - 64
    gen = torch.Generator(device=DEV).manual_seed(0)
    # entry j of a row lies in band j of the columns: ascending within the row, as a transpose produces them
    col = torch.randint(0, band, (m, per_row), dtype=torch.int32, device=DEV, generator=gen)
    col += (torch.arange(per_row, dtype=torch.int32, device=DEV) * band)[None, :]
    col = col.reshape(-1)
    val = torch.rand(nnz, device=DEV, generator=gen)
    rowptr = (torch.arange(m + 1, dtype=torch.int64, device=DEV) * per_row).to(torch.int32)
    assert int(rowptr[-1]) == nnz
    a = ops.CsrMatrix(rowptr, col, val, (m, k), seg_len=512)
    assert a.n_long_rows == m and a.n_segments == 2 * m
    h = torch.randn(k, d, device=DEV, generator=gen)
    y = ops.spmm(a, h)
    block = 2 ** 16
    worst, largest = 0.0, 0.0
    for r0 in range(0, m, block):
        c = col[r0 * per_row:(r0 + block) * per_row].long()
        ref = (h[c].double().view(block, per_row, d) * val[r0 * per_row:(r0 + block) * per_row].double().view(block, per_row, 1)).sum(1)
        worst = max(worst, (y[r0:r0 + block].double() - ref).abs().max().item())
        largest = max(largest, ref.abs().max().item())
        del c, ref
    print("max error %.3e of %.3e" % (worst, largest), flush=True)
    assert worst <= FP32_TOL * largest
    at = ops.csr_transpose(a, seg_len=4096)
    assert at.shape == (k, m) and at.nnz == nnz
    gm = torch.randn(m, d, device=DEV, generator=gen)
    lhs = (y.double() * gm.double()).sum().item()
    rhs = (h.double() * ops.spmm(at, gm).double()).sum().item()
    assert abs(lhs - rhs) <= 1e-5 * (y.double().norm() * gm.double().norm()).item()
    att = ops.csr_transpose(at)
    assert torch.equal(att.rowptr, a.rowptr) and torch.equal(att.col, a.col) and torch.equal(att.val, a.val)


def test_spmm_int64_torch_csr_and_chunked_equivalence():
    say("spmm from torch CSR tensor; chunked == unchunked")
    g = graph_small(n=900, pairs=9000, seed=3)
    a_t = g.torch_csr().to(DEV)
    h = torch.randn(900, 32, generator=torch.Generator().manual_seed(1))
    y = ops.spmm(a_t, h.to(DEV)).cpu()
    assert getattr(a_t, "_plexus_amd_csr", None) is not None  # converted once, cached
    assert rel_err(y, po.spmm(g.torch_csr(), h)) <= FP32_TOL
    # row-chunked aggregation of the reference (gcn_conv.py:67-128) gives the same rows
    ref_chunked = po.chunked_spmm(g.torch_csr(), h, max_rows_per_chunk=250)
    assert rel_err(y, ref_chunked) <= FP32_TOL


def test_spmm_bf16():
    say("spmm bf16 storage")
    g = S.build_graph(2000, "chunglu", 30000, seed=4, device="cpu")
    for d in (256, 64, 100, 6):
        h = torch.randn(2000, d, generator=torch.Generator().manual_seed(d)).to(torch.bfloat16)
        a = to_dev(g, seg_len=128)
        y = ops.spmm(a, h.to(DEV))
        assert y.dtype == torch.bfloat16
        ref = oracle_spmm64(g, h.float())  # fp32 math on bf16-rounded inputs
        assert rel_err(y.float().cpu(), ref) <= BF16_TOL
        # accumulation is fp32: the only error is the final rounding, 2^-9 relative per element
        assert rel_err(y.float().cpu(), ref) <= 2.0 ** -8


GEMM_SHAPES = [(1, 1, 1), (5, 3, 2), (127, 16, 33), (128, 32, 32), (300, 47, 128), (1000, 128, 100), (513, 128, 128),
               (260, 7, 16), (200, 16, 1433), (150, 256, 256), (64, 130, 70)]


@pytest.fixture(params=["split", "mfma32"])
def fp32_gemm_path(request):
    """Both implementations of the fp32 products: exact three-way bf16 splits on the bf16 matrix cores (taken when
    the operands are aligned for it) and the fp32 MFMA kernels."""
    keep = ops.SPLIT_GEMM
    ops.SPLIT_GEMM = request.param == "split"
    yield request.param
    ops.SPLIT_GEMM = keep


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES + [(3000, 128, 96), (777, 48, 128), (2049, 200, 40)])
def test_gemm_nn(m, n, k, fp32_gemm_path):
    say("gemm_nn %dx%dx%d %s" % (m, n, k, fp32_gemm_path))
    gen = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=gen)
    b = torch.randn(k, n, generator=gen)
    c = ops.gemm_nn(a.to(DEV), b.to(DEV)).cpu()
    ref = oracle_c.gemm(a.numpy(), b.numpy())
    assert rel_err(c, ref) <= FP32_TOL
    assert rel_err(c, torch.mm(a, b)) <= FP32_TOL  # the reference's operator
    cr = ops.gemm_nn(a.to(DEV), b.to(DEV), relu=True).cpu()
    assert rel_err(cr, np.maximum(ref, 0)) <= FP32_TOL and (cr >= 0).all()


def test_split_gemm_is_taken_and_keeps_fp32_accuracy_on_hard_inputs():
    """The split path must not lose what an fp32 product keeps: operands spanning many binades, exact small
    integers, a column slice as output, and the workspace / alignment contract."""
    say("split gemm: wide dynamic range, exact integers, contract")
    from plexus_amd import _lib

    gen = torch.Generator().manual_seed(7)
    m, k, n = 2000, 128, 64
    a = torch.randn(m, k, generator=gen) * torch.exp2(torch.randint(-20, 20, (m, 1), generator=gen).float())
    b = torch.randn(k, n, generator=gen) * torch.exp2(torch.randint(-20, 20, (1, n), generator=gen).float())
    ref = a.double() @ b.double()
    got = ops.gemm_nn(a.to(DEV), b.to(DEV)).cpu().double()
    # row- and column-scaled data: compare element-wise against the scale of each dot product
    scale = (a.double().abs() @ b.double().abs())
    err_split = ((got - ref).abs() / scale).max().item()
    keep, ops.SPLIT_GEMM = ops.SPLIT_GEMM, False
    err_mfma32 = ((ops.gemm_nn(a.to(DEV), b.to(DEV)).cpu().double() - ref).abs() / scale).max().item()
    ops.SPLIT_GEMM = keep
    assert err_split <= 16 * 2.0 ** -24 and err_split <= 2 * err_mfma32  # the level of an fp32 accumulation over K = 128
    ai = torch.randint(-50, 50, (m, k), generator=gen).float()
    bi = torch.randint(-50, 50, (k, n), generator=gen).float()
    assert torch.equal(ops.gemm_nn(ai.to(DEV), bi.to(DEV)).cpu(), ai @ bi)  # integer products below 2^24 are exact
    wide = torch.zeros(m, n + 8, device=DEV)
    ops.gemm_nn(ai.to(DEV), bi.to(DEV), out=wide[:, 3:3 + n])
    assert torch.equal(wide[:, 3:3 + n].cpu(), ai @ bi) and (wide[:, :3] == 0).all() and (wide[:, 3 + n:] == 0).all()
    lib = _lib.load()
    need = int(lib.plx_gemm_f32_split_workspace_bytes(n, k))
    assert need == 3 * 64 * 128 * 2 + 256  # three bf16 planes of the weight and the flag words of the Inf / NaN check
    ad, bd, cd = ai.to(DEV), bi.to(DEV), torch.empty(m, n, device=DEV)
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.plx_gemm_nn_f32_split(m, n, k, ad.data_ptr(), k, bd.data_ptr(), n, cd.data_ptr(), n, 0, ws.data_ptr(), need - 1, stream) == _lib.PLX_ERR_WORKSPACE
    # weights up to 128 x 128: any alignment and any K (element loads); beyond that the operands must allow 64-bit loads
    assert lib.plx_gemm_nn_f32_split(m - 1, n, k - 3, ad.data_ptr() + 4, k, bd.data_ptr(), n, cd.data_ptr(), n, 0, ws.data_ptr(), need, stream) == 0
    flat = ai.reshape(-1)[1:1 + (m - 1) * k].reshape(m - 1, k)[:, :k - 3]
    assert torch.equal(cd[:m - 1].cpu(), flat @ bi[:k - 3])
    k2, n2 = 256, 136
    a2, b2, c2 = torch.zeros(m * k2 + 4, device=DEV), torch.zeros(k2, n2, device=DEV), torch.empty(m, n2, device=DEV)
    need2 = int(lib.plx_gemm_f32_split_workspace_bytes(n2, k2))
    ws2 = torch.empty(need2, dtype=torch.uint8, device=DEV)
    assert lib.plx_gemm_nn_f32_split(m, n2, k2, a2.data_ptr() + 4, k2, b2.data_ptr(), n2, c2.data_ptr(), n2, 0, ws2.data_ptr(), need2, stream) == _lib.PLX_ERR_INVALID
    assert lib.plx_gemm_nn_f32_split(m, n2, k2 - 3, a2.data_ptr(), k2, b2.data_ptr(), n2, c2.data_ptr(), n2, 0, ws2.data_ptr(), need2, stream) == _lib.PLX_ERR_INVALID
    assert lib.plx_gemm_nn_f32_split(m, n2, k2 - 2, a2.data_ptr() + 8, k2, b2.data_ptr(), n2, c2.data_ptr(), n2, 0, ws2.data_ptr(), need2, stream) == 0


@pytest.mark.parametrize("k,n", [(128, 128), (100, 47), (256, 256), (602, 130)])  # resident kernel, chunked kernel, 64-bit loads
def test_fp32_products_with_inf_nan_and_values_near_overflow_agree_with_torch(k, n):
    """Inf, NaN and finite values whose bf16 rounding would overflow, in either operand: the default (split) products
    give what torch.mm gives -- Inf where it gives Inf, NaN where NaN, the same finite numbers elsewhere."""
    say("fp32 products with Inf / NaN / 3.4e38, K=%d N=%d" % (k, n))
    gen = torch.Generator().manual_seed(k + n)
    m = 700
    big = 3.4e38  # above 0x7f7f8000: rounds to Inf in bf16
    a0 = torch.randn(m, k, generator=gen)
    w0 = torch.randn(k, n, generator=gen) * 0.1

    def same(got, ref, what):
        got, ref = got.cpu(), ref.cpu()
        assert torch.equal(torch.isnan(got), torch.isnan(ref)), what + ": NaN pattern"
        assert torch.equal(torch.isinf(got), torch.isinf(ref)) and torch.equal(got[torch.isinf(ref)], ref[torch.isinf(ref)]), what + ": Inf pattern"
        fin = torch.isfinite(ref)
        assert rel_err(got[fin], ref[fin]) <= FP32_TOL, what

    def both_paths(fn):
        keep = ops.SPLIT_GEMM
        try:
            ops.SPLIT_GEMM = True
            y_split = fn()
            ops.SPLIT_GEMM = False
            y_mfma = fn()
        finally:
            ops.SPLIT_GEMM = keep
        return y_split, y_mfma

    cases = []
    # the large operand: one special value per row, in rows 0..3 (the rest of row 1 cleared: whether a sum of finite
    # terms next to 3.4e38 overflows depends on the order of summation)
    a = a0.clone()
    a[1, :] = 0.0
    a[0, 3], a[1, 5], a[2, 7], a[3, 9] = float("inf"), big, float("nan"), float("-inf")
    cases.append(("special values in A", a, w0))
    # finite but huge everywhere in one row: no Inf may appear that fp32 does not produce
    a = a0.clone()
    a[10, :] = 0.0
    a[10, 1] = big
    a[11, :] = 0.0
    a[11, 2] = -big
    w = w0.clone()
    w[1, :] = 0.5
    w[2, :] = 2.0  # -3.4e38 * 2 overflows to -Inf in fp32 as well
    cases.append(("huge finite values", a, w))
    # the small operand
    w = w0.clone()
    w[2, 1], w[4, 3] = float("inf"), float("nan")
    w[6, 5] = big
    a = a0.clone()
    a[:, 6] = a[:, 6].clamp(-0.9, 0.9)  # 3.4e38 * a stays finite; the other terms of these sums are tiny beside it
    cases.append(("special values in W", a, w))
    for what, a, w in cases:
        ad, wd = a.to(DEV), w.to(DEV)
        ref = torch.mm(ad, wd)
        y_split, y_mfma = both_paths(lambda: ops.gemm_nn(ad, wd))
        same(y_split, ref, what + " (NN, split)")
        same(y_mfma, ref, what + " (NN, fp32 MFMA)")
        same(y_split, torch.mm(a, w), what + " (NN, split vs host)")
        # NT form with the ReLU mask: GRAD_AGG = (G * [mask > 0]) . W^T with W stored (n_out = k here, n_in = n): use W^T of the above
        wt = wd.t().contiguous()  # [n, k]
        mask = torch.randn(m, k, generator=gen).to(DEV)
        mask[0:12] = 1.0  # keep the special rows
        ref_nt = torch.mm(torch.where(mask > 0, ad, torch.zeros_like(ad)), wt.t())
        z_split, z_mfma = both_paths(lambda: ops.gemm_nt(ad, wt, mask=mask))
        same(z_split, ref_nt, what + " (NT + mask, split)")
        same(z_mfma, ref_nt, what + " (NT + mask, fp32 MFMA)")
        # a special value under a zero of the mask does not exist for the product
        mask2 = mask.clone()
        mask2[0:12] = -1.0
        clean = torch.where(mask2 > 0, ad, torch.zeros_like(ad))
        z2, _ = both_paths(lambda: ops.gemm_nt(ad, wt, mask=mask2))
        same(z2, torch.mm(clean, wt.t()), what + " (NT, special rows masked out)")
    # and a clean product right after a flagged one (the flag words are cleared per call)
    y_split, _ = both_paths(lambda: ops.gemm_nn(a0.to(DEV), w0.to(DEV)))
    assert torch.isfinite(y_split).all() and rel_err(y_split, torch.mm(a0, w0)) <= FP32_TOL


@pytest.mark.parametrize("m,n,k", [(1500, 128, 602), (700, 200, 150), (333, 130, 258)])
def test_split_gemm_with_64_bit_loads(m, n, k):
    """Contraction lengths that are even but not multiples of 4 (rows of 602 elements are 8-byte aligned only): the
    split kernels read them with pairs of 64-bit loads."""
    say("split gemm, K %% 4 == 2: %dx%dx%d" % (m, n, k))
    assert ops.SPLIT_GEMM and k % 4 == 2
    gen = torch.Generator().manual_seed(k)
    a, w, g = torch.randn(m, k, generator=gen), torch.randn(k, n, generator=gen), torch.randn(m, n, generator=gen)
    assert ops._split_ok(n, k, a.to(DEV))
    out = ops.gemm_nn(a.to(DEV), w.to(DEV), relu=True).cpu()
    assert rel_err(out, torch.relu(a.double() @ w.double())) <= FP32_TOL
    mask = torch.relu(torch.randn(m, n, generator=gen))
    dagg = ops.gemm_nt(g.to(DEV), w.to(DEV), mask=mask.to(DEV)).cpu()  # contraction over n: aligned or not, as n falls
    assert rel_err(dagg, (g.double() * (mask > 0)) @ w.double().t()) <= FP32_TOL
    # contraction over k with a mask of k columns
    g2, mask2 = torch.randn(m, k, generator=gen), torch.relu(torch.randn(m, k, generator=gen))
    out2 = ops.gemm_nt(g2.to(DEV), w.t().contiguous().to(DEV), mask=mask2.to(DEV)).cpu()
    assert rel_err(out2, (g2.double() * (mask2 > 0)) @ w.double()) <= FP32_TOL


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES + [(3000, 128, 96), (777, 48, 128), (2049, 200, 40)])
def test_gemm_nt_and_mask(m, n, k, fp32_gemm_path):
    say("gemm_nt %dx%dx%d %s" % (m, n, k, fp32_gemm_path))
    gen = torch.Generator().manual_seed(m * 3 + n + k)
    g = torch.randn(m, k, generator=gen)
    w = torch.randn(n, k, generator=gen)
    c = ops.gemm_nt(g.to(DEV), w.to(DEV)).cpu()
    assert rel_err(c, oracle_c.gemm(g.numpy(), w.numpy(), tb=True)) <= FP32_TOL
    assert rel_err(c, torch.mm(g, torch.t(w))) <= FP32_TOL
    act = torch.relu(torch.randn(m, k, generator=gen))
    cm = ops.gemm_nt(g.to(DEV), w.to(DEV), mask=act.to(DEV)).cpu()
    ref = oracle_c.gemm((g * (act > 0)).numpy(), w.numpy(), tb=True)
    assert rel_err(cm, ref) <= FP32_TOL


def _pack_bits(x):
    """Reference of the sign bits: bit c % 32 of int32 word [row, c // 32] is x[row, c] > 0."""
    m, n = x.shape
    words = (n + 31) // 32
    pos = torch.zeros(m, words * 32, dtype=torch.int64)
    pos[:, :n] = (x > 0).to(torch.int64)
    w = (pos.reshape(m, words, 32) << torch.arange(32, dtype=torch.int64)).sum(-1)
    return torch.where(w >= 2**31, w - 2**32, w).to(torch.int32)


@pytest.mark.parametrize("m,n,k", [(3000, 128, 100), (1001, 128, 128), (777, 47, 128), (2050, 100, 64), (500, 200, 150), (33, 7, 5)])
def test_relu_mask_as_sign_bits(m, n, k, fp32_gemm_path):
    say("sign bits of a product and a bit mask into the next, M=%d N=%d K=%d (%s)" % (m, n, k, fp32_gemm_path))
    gen = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=gen).to(DEV)
    w = torch.randn(k, n, generator=gen).to(DEV) * 0.1
    # forward: the product writes the bits of its own result (fused in the kernel for weights up to 128 x 128)
    out, bits = ops.gemm_nn(a, w, relu=True, want_bits=True)
    assert torch.equal(out, ops.gemm_nn(a, w, relu=True))
    assert bits.dtype == torch.int32 and tuple(bits.shape) == (m, (n + 31) // 32)
    assert torch.equal(bits.cpu(), _pack_bits(out.cpu()))
    assert torch.equal(ops.sign_bits(out), bits)
    assert 0.3 < (out > 0).float().mean().item() < 0.7  # a real mask, not all ones
    # backward: GRAD_AGG = (G * mask) . W^T with the mask as bits gives the bits of the fp32 mask
    gout = torch.randn(m, n, generator=gen).to(DEV)
    want = ops.gemm_nt(gout, w, mask=out)
    got = ops.gemm_nt(gout, w, mask=out, mask_bits=bits)
    assert torch.equal(got, want)
    ref = (gout.cpu().double() * (out.cpu() > 0)) @ w.cpu().double().T
    assert rel_err(got.cpu(), ref) <= FP32_TOL
    # a view with a row pitch that 128-bit loads cannot take: the fp32 mask is read instead, same result
    wide = torch.zeros(m, n + 3, device=DEV)
    wide[:, 1:n + 1] = gout
    view = wide[:, 1:n + 1]
    assert torch.equal(ops.gemm_nt(view, w, mask=out, mask_bits=bits), ops.gemm_nt(view, w, mask=out))
    with pytest.raises(ValueError):
        ops.gemm_nt(gout, w, mask_bits=bits)  # the bits stand for a mask that must be given too


@pytest.mark.parametrize("n", [70, 96, 33, 128])
def test_sign_bits_through_the_raw_entry_point_with_the_smallest_pitch(n):
    """N in 65..96 runs four column tiles but a row holds three words: with a pitch of exactly ceil(N / 32) words the
    fourth tile must not write (it would land on the next row's first word, and past the buffer after the last row)."""
    say("sign bits with ldw = ceil(N / 32), N=%d" % n)
    from plexus_amd import _lib

    lib = _lib.load()
    m, k = 1000 + 7, 64
    words = (n + 31) // 32
    gen = torch.Generator().manual_seed(n)
    a = torch.randn(m, k, generator=gen).to(DEV)
    w = (torch.randn(k, n, generator=gen) * 0.1).to(DEV)
    c = torch.empty(m, n, device=DEV)
    guard = 0x5A5A5A5A
    bits = torch.full((m * words + 8,), guard, dtype=torch.int32, device=DEV)  # rows packed back to back, guard words behind
    need = int(lib.plx_gemm_f32_split_workspace_bytes(n, k))
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    _lib.check(lib.plx_gemm_nn_f32_split_bits(m, n, k, a.data_ptr(), k, w.data_ptr(), n, c.data_ptr(), n, _lib.PLX_GEMM_RELU,
                                              bits.data_ptr(), words, ws.data_ptr(), need, torch.cuda.current_stream().cuda_stream),
               "plx_gemm_nn_f32_split_bits")
    assert torch.equal(bits[: m * words].reshape(m, words).cpu(), _pack_bits(c.cpu()))
    assert (bits[m * words:] == guard).all()
    assert 0.3 < (c > 0).float().mean().item() < 0.7


def test_sign_bits_follow_the_product_the_guarded_launch_redoes():
    say("sign bits when an operand holds Inf (the fp32 kernel redoes the product)")
    gen = torch.Generator().manual_seed(9)
    a = torch.randn(700, 128, generator=gen)
    a[5, 3] = float("inf")
    a[9, 7] = float("nan")
    w = torch.randn(128, 128, generator=gen) * 0.1
    out, bits = ops.gemm_nn(a.to(DEV), w.to(DEV), relu=True, want_bits=True)
    assert torch.isinf(out[5]).any() or torch.isnan(out[5]).any()
    assert torch.equal(bits.cpu(), _pack_bits(out.cpu()))


# (40000, 47, 128), (50001, 33, 100), (3000, 7, 64): B in rows without 16-byte alignment, read element by element by the split kernel
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES + [(70000, 128, 100), (40000, 47, 128), (30011, 128, 128), (5000, 200, 150), (2500, 64, 300),
                                                   (31, 128, 128), (1, 5, 3), (50001, 33, 100), (3000, 7, 64)])
def test_gemm_tn_and_mask(m, n, k, fp32_gemm_path):
    say("gemm_tn %dx%dx%d %s" % (m, n, k, fp32_gemm_path))
    gen = torch.Generator().manual_seed(m * 5 + n + k)
    a = torch.randn(m, k, generator=gen)
    g = torch.randn(m, n, generator=gen)
    c = ops.gemm_tn(a.to(DEV), g.to(DEV)).cpu()
    assert c.shape == (k, n)
    ref = oracle_c.gemm(a.numpy(), g.numpy(), ta=True)
    assert rel_err(c, ref) <= FP32_TOL
    act = torch.relu(torch.randn(m, n, generator=gen))
    cm = ops.gemm_tn(a.to(DEV), g.to(DEV), mask=act.to(DEV)).cpu()
    assert rel_err(cm, oracle_c.gemm(a.numpy(), (g * (act > 0)).numpy(), ta=True)) <= FP32_TOL
    # run-to-run bit reproducibility (no atomics, fixed order)
    assert torch.equal(c, ops.gemm_tn(a.to(DEV), g.to(DEV)).cpu())
    # the mask as one bit per element, and the factor of a dropout layer
    bits = ops.sign_bits(act.to(DEV))
    assert torch.equal(ops.gemm_tn(a.to(DEV), g.to(DEV), mask=act.to(DEV), mask_bits=bits).cpu(), cm)
    c2 = ops.gemm_tn(a.to(DEV), g.to(DEV), mask=act.to(DEV), mask_bits=bits, alpha=2.0).cpu()
    assert torch.equal(c2, 2.0 * cm)
    # operands inside wider matrices, off 16-byte boundaries: element loads, same numbers as the oracle
    wide_a = torch.zeros(m, k + 5)
    wide_a[:, 3:3 + k] = a
    wide_g = torch.zeros(m, n + 2)
    wide_g[:, 1:1 + n] = g
    cv = ops.gemm_tn(wide_a.to(DEV)[:, 3:3 + k], wide_g.to(DEV)[:, 1:1 + n], mask=act.to(DEV), mask_bits=bits).cpu()
    assert rel_err(cv, oracle_c.gemm(a.numpy(), (g * (act > 0)).numpy(), ta=True)) <= FP32_TOL


def test_gemm_tn_split_keeps_fp32_accuracy_over_millions_of_rows_and_handles_nonfinite_values():
    say("gemm_tn split: long sums, hard values, Inf / NaN")
    gen = torch.Generator().manual_seed(77)
    m, n, k = 1 << 20, 128, 128
    a = torch.randn(m, k, generator=gen)
    g = torch.randn(m, n, generator=gen) * torch.exp2(torch.randint(-20, 20, (m, 1), generator=gen).float())  # rows spanning 40 binades
    ad, gd = a.to(DEV), g.to(DEV)
    c = ops.gemm_tn(ad, gd).cpu()
    ref = (a.double().T @ g.double())
    keep = ops.SPLIT_GEMM
    ops.SPLIT_GEMM = False
    c32 = ops.gemm_tn(ad, gd).cpu()
    ops.SPLIT_GEMM = keep
    e_split, e_mfma = rel_err(c, ref), rel_err(c32, ref)
    print("rel err vs fp64: split %.2e, fp32 MFMA %.2e" % (e_split, e_mfma), flush=True)
    assert e_split <= 2e-6 and e_split <= 4 * e_mfma + 1e-7
    # exact small integers: every piece product and every partial sum is exact in fp32
    ai = torch.randint(-3, 4, (4096, 100), generator=gen).float()
    gi = torch.randint(-3, 4, (4096, 47), generator=gen).float()
    assert torch.equal(ops.gemm_tn(ai.to(DEV), gi.to(DEV)).cpu(), (ai.double().T @ gi.double()).float())
    # Inf / NaN in either operand: what torch.mm gives (the fp32 kernel redoes the product)
    for where in ("a", "g"):
        a2, g2 = a[:5000].clone(), torch.randn(5000, n, generator=gen)
        (a2 if where == "a" else g2)[17, 5] = float("inf")
        (a2 if where == "a" else g2)[99, 7] = float("nan")
        got = ops.gemm_tn(a2.to(DEV), g2.to(DEV)).cpu()
        want = torch.mm(a2.t(), g2)
        assert torch.equal(torch.isnan(got), torch.isnan(want)) and torch.equal(torch.isinf(got), torch.isinf(want))
        fin = torch.isfinite(want)
        assert rel_err(got[fin], want[fin].double()) <= FP32_TOL


def test_gemm_strided_views_and_tuned_matmul():
    say("gemm with leading dimensions; tuned_matmul routing")
    from plexus_amd.utils.matmul_tuning import tuned_matmul

    gen = torch.Generator().manual_seed(0)
    big = torch.randn(300, 90, generator=gen)
    a = big.to(DEV)[:, 10:75]  # ld 90, width 65, unaligned start
    b = torch.randn(65, 33, generator=gen)
    assert rel_err(ops.gemm_nn(a, b.to(DEV)).cpu(), big[:, 10:75] @ b) <= FP32_TOL
    agg = torch.randn(400, 24, generator=gen)
    go = torch.randn(400, 12, generator=gen)
    w = torch.randn(24, 12, generator=gen)
    assert rel_err(tuned_matmul(torch.t(agg.to(DEV)), go.to(DEV), "AGG.T * GRAD_OUT 0").cpu(), agg.t() @ go) <= FP32_TOL
    assert rel_err(tuned_matmul(go.to(DEV), torch.t(w.to(DEV)), "GRAD_OUT * W.T 0").cpu(), go @ w.t()) <= FP32_TOL
    assert rel_err(tuned_matmul(agg.to(DEV), w.to(DEV), "AGG * W 0").cpu(), agg @ w) <= FP32_TOL


def test_relu_kernels():
    say("relu fwd/bwd")
    gen = torch.Generator().manual_seed(0)
    for shape in [(33, 7), (128, 128), (5, 1)]:
        x = torch.randn(*shape, generator=gen)
        dy = torch.randn(*shape, generator=gen)
        y = ops.relu(x.to(DEV))
        assert torch.equal(y.cpu(), torch.relu(x))
        dx = ops.relu_bwd(dy.to(DEV), y)
        assert torch.equal(dx.cpu(), dy * (x > 0))


@pytest.mark.parametrize("m,c", [(1, 1), (10, 7), (1000, 47), (333, 64), (257, 100), (50, 1000), (4100, 16), (1031, 41), (2055, 63),
                                 (777, 3), (515, 33)])
def test_softmax_xent(m, c):
    say("softmax_xent %dx%d" % (m, c))
    gen = torch.Generator().manual_seed(m + c)
    logits = torch.randn(m, c, generator=gen) * 3
    y = torch.randint(0, c, (m,), generator=gen)
    loss, dl = ops.softmax_xent(logits.to(DEV), y.to(DEV), m, c)
    rl, rs, ro = po.cross_entropy_forward(logits, y, m, c)  # the reference's operator chain on the host
    rg = po.cross_entropy_backward(rs, ro.float(), m)
    closs, cgrad = oracle_c.softmax_xent(logits.numpy(), y.numpy(), m, c)
    assert abs(loss.item() - closs) <= FP32_TOL * abs(closs)
    assert abs(loss.item() - rl.item()) <= FP32_TOL * abs(closs)
    assert rel_err(dl.cpu(), cgrad) <= FP32_TOL
    assert rel_err(dl.cpu(), rg) <= FP32_TOL
    # library closed form: equals F.cross_entropy when every label is valid
    assert abs(loss.item() - torch.nn.functional.cross_entropy(logits.double(), y).item()) <= FP32_TOL * abs(closs)


@pytest.mark.parametrize("c", [12, 13])  # even: padded-tile kernel; odd: contiguous-copy kernel
def test_softmax_xent_special_cases_and_no_mutation(c):
    say("softmax_xent masks, padding, gscale, C=%d" % c)
    gen = torch.Generator().manual_seed(9)
    m = 40
    logits = torch.randn(m, c, generator=gen)
    y = torch.randint(0, 10, (m,), generator=gen)
    y[3] = -1
    y[7] = 11  # labelled with a padded class
    y[9] = 50  # outside [0, C)
    num_nodes, num_classes = 36, 10
    ld, yd = logits.to(DEV), y.to(DEV)
    keep_l, keep_y = ld.clone(), yd.clone()
    loss, dl = ops.softmax_xent(ld, yd, num_nodes, num_classes, gscale=2.5)
    assert torch.equal(ld, keep_l) and torch.equal(yd, keep_y)
    closs, cgrad = oracle_c.softmax_xent(logits.numpy(), y.numpy(), num_nodes, num_classes, gscale=2.5)
    assert abs(loss.item() - closs) <= FP32_TOL * abs(closs)
    assert rel_err(dl.cpu(), cgrad) <= FP32_TOL
    assert (dl[3] == 0).all()  # negative label: no gradient
    assert (dl[:, 10:] == 0)[y != 11].all()  # padded classes carry no probability
    assert (dl[36:].cpu()[torch.arange(4), y[36:]] < 0).all() and loss.item() > 4 * 20.7 / 36
    # row offset shifts the padded-row test
    loss2, _ = ops.softmax_xent(ld, yd, num_nodes, num_classes, row_offset=30)
    assert loss2.item() > loss.item()
    # the same rows as a strided view of a wider matrix (leading dimension > C)
    wide = torch.zeros(m, c + 5, device=DEV)
    wide[:, :c] = ld
    loss3, dl3 = ops.softmax_xent(wide[:, :c], yd, num_nodes, num_classes, gscale=2.5)
    assert abs(loss3.item() - closs) <= FP32_TOL * abs(closs) and rel_err(dl3.cpu(), cgrad) <= FP32_TOL


def test_upstream_scalar_and_standalone_relu_run_on_the_library():
    say("loss scaled upstream; ReLU outside the layer")
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.train import relu

    gen = torch.Generator().manual_seed(5)
    for n, dtype in ((1000 * 48, torch.float32), (1003, torch.float32), (4096, torch.bfloat16), (77, torch.bfloat16)):
        x = torch.randn(n, generator=gen).to(dtype)
        got = ops.scale_by_scalar(x.to(DEV), torch.tensor(-2.5, device=DEV))
        assert got.dtype == dtype and torch.equal(got.cpu(), (x.float() * -2.5).to(dtype))
    m, c = 1500, 47
    logits = torch.randn(m, c, generator=gen)
    y = torch.randint(0, c, (m,), generator=gen)
    ld = relu(logits.to(DEV).requires_grad_())  # a non-leaf: the gradient flows through relu's backward kernel
    leaf = ld.grad_fn.next_functions[0][0].variable
    (parallel_cross_entropy(ld, y.to(DEV), 1, m, c) * 3.0).backward()
    ref = logits.clone().requires_grad_()
    (torch.nn.functional.cross_entropy(torch.relu(ref), y) * 3.0).backward()
    assert rel_err(leaf.grad, ref.grad) <= FP32_TOL
    with pytest.raises(TypeError):
        ops.relu(logits.to(DEV).to(torch.bfloat16))


def test_gcn_norm_kernel():
    say("gcn_norm_csr")
    g = S.build_graph(1500, "chunglu", 12000, seed=5, device="cpu")
    ones = torch.ones_like(g.val)
    a = ops.CsrMatrix(g.rowptr.to(DEV), g.col.to(DEV), ones.to(DEV), g.shape)
    v = ops.gcn_norm_csr(a).cpu()
    assert rel_err(v, po.gcn_norm_csr_values(g.rowptr, g.col, ones)) <= FP32_TOL
    assert rel_err(v, oracle_c.gcn_norm_csr(g.rowptr.numpy(), g.col.numpy(), ones.numpy())) <= FP32_TOL
    assert rel_err(v, g.val) <= FP32_TOL


def test_layer_forward_backward_matches_oracle():
    say("GCNConv layer fwd+bwd, fused and unfused ReLU")
    from plexus_amd.gcn_conv import GCNConv

    n, din, dout = 1200, 100, 47
    g = S.build_graph(n, "chunglu", 15000, seed=6, device="cpu")
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n * din, generator=gen)  # flat, as layer 0 receives it
    w = po.kaiming_uniform_weight(din, dout, gen)
    go = torch.randn(n, dout, generator=gen)
    out_ref, agg_ref = po.gcn_conv_forward(x, g.torch_csr(), w, (n, din), (din, dout))
    gx_ref, gw_ref = po.gcn_conv_backward(go, agg_ref, w, g.torch_csr(True), (din, dout), flatten_grad_x=True)

    shards = [(to_dev(g), to_dev(g, True))]
    layer = GCNConv(din, dout, 0, weight=w)
    xd = x.to(DEV).requires_grad_()
    out = layer(xd, shards)
    out.backward(go.to(DEV))
    assert rel_err(out, out_ref) <= FP32_TOL
    assert xd.grad.shape == x.shape and rel_err(xd.grad, gx_ref) <= FP32_TOL
    assert layer.weight.grad.shape == w.shape and rel_err(layer.weight.grad, gw_ref) <= FP32_TOL

    # fused ReLU: forward max(OUT, 0); backward masks GRAD_OUT by OUT > 0
    layer2 = GCNConv(din, dout, 1, weight=w, fuse_relu=True)
    xd2 = x.reshape(n, din).to(DEV).requires_grad_()
    out2 = layer2(xd2, shards)
    out2.backward(go.to(DEV))
    gmask = go * (out_ref > 0)
    gx2_ref, gw2_ref = po.gcn_conv_backward(gmask, agg_ref, w, g.torch_csr(True), (din, dout))
    assert rel_err(out2, torch.relu(out_ref)) <= FP32_TOL
    assert rel_err(xd2.grad, gx2_ref) <= FP32_TOL and rel_err(layer2.weight.grad, gw2_ref) <= FP32_TOL


@pytest.mark.parametrize("fuse_relu", [True, False])
def test_config1_ten_epoch_loss_curve(fuse_relu):
    """2-layer GCN of the CPU-runnable configuration: ten AdamW epochs against the oracle's."""
    say("config 1, 10 epochs, fuse_relu=%s" % fuse_relu)
    from plexus_amd.train import Net, make_optimizer, run_epochs

    g, x, y, dims = S.config1(device="cpu", seed=0)
    weights = S.glorot_weights(dims, seed=0)
    n = g.shape[0]
    ref_losses, ref_x, ref_w = po.train_epochs(x, weights, dims, [(g.torch_csr(), g.torch_csr(True))], y, n, 7, epochs=10)
    ref64, x64, w64 = po.train_epochs(x.double(), [w.double() for w in weights], dims,
                                      [(g.torch_csr().double(), g.torch_csr(True).double())], y, n, 7, epochs=10)

    model = Net(2, dims[0], dims[1], dims[2], weights=weights, fuse_relu=fuse_relu)
    feats = x.reshape(-1).to(DEV).requires_grad_()
    opt = make_optimizer(model, feats)
    shards = [(g.torch_csr().to(DEV), g.torch_csr(True).to(DEV))]
    masks = []  # the ReLU mask of every epoch, for the comparison of the trained tensors below
    model.layers[0].register_forward_hook(lambda mod, args, out: masks.append((out.detach() > 0).cpu()))
    losses = run_epochs(model, opt, feats, shards, y.to(DEV), n, 7, 10)
    import json
    import os
    golden = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1_golden.json")))
    assert g.nnz == golden["nnz"]
    for l, want in zip(losses, golden["losses_fp64"]):  # the committed fp64 loss curve of the oracle
        assert abs(l - want) <= FP32_TOL * abs(want)
    print("gpu   ", ["%.6f" % v for v in losses], flush=True)
    print("oracle", ["%.6f" % v for v in ref_losses], flush=True)
    for l, r, r64 in zip(losses, ref_losses, ref64):
        assert abs(l - r64) <= FP32_TOL * abs(r64) or abs(l - r) <= FP32_TOL * abs(r)
    assert losses[-1] < losses[0]
    # The trained tensors.  A hidden unit whose pre-activation is within rounding of zero can take either side of the ReLU in
    # two fp32 summation orders, and Adam turns the gradient that then appears or vanishes into a step of +-lr for every
    # feature of that vertex's neighbours; so the oracle's backward passes are given the masks the GPU run produced, and
    # the trained features and weights must then agree like any other fp32 tensor.
    picked = lambda e: [masks[e], None]
    pair = [(g.torch_csr(), g.torch_csr(True))]
    pair64 = [(g.torch_csr().double(), g.torch_csr(True).double())]
    p32, px32, pw32 = po.train_epochs(x, weights, dims, pair, y, n, 7, epochs=10, masks_of_epoch=picked)
    p64, px64, pw64 = po.train_epochs(x.double(), [w.double() for w in weights], dims, pair64, y, n, 7, epochs=10, masks_of_epoch=picked)
    assert max(abs(u - v) for u, v in zip(p64, ref64)) <= 1e-6
    assert_parity(feats, px32, px64, what="trained features")
    for i, layer in enumerate(model.layers):
        # an element of GRAD_W that cancels to the size of Adam's eps is moved by rounding noise: 1e-4 of the largest weight
        assert_parity(layer.weight, pw32[i], pw64[i], tol=1e-4, what="trained weight %d" % i)


def oracle_rows_of_spmm(g, h):
    """(row ids, rows of A.H by the fp64-accumulating oracle) for the 8 longest, the 8 shortest and 200 random rows of a
    graph held on the device; only the entries of those rows leave the device."""
    m = g.shape[0]
    deg = (g.rowptr[1:] - g.rowptr[:-1]).cpu()
    pick = torch.cat([torch.topk(deg, 8).indices, torch.topk(-deg, 8).indices,
                      torch.randint(0, m, (200,), generator=torch.Generator().manual_seed(0))])
    sub_counts = deg[pick]
    sub_rowptr = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(sub_counts, 0)])
    starts = g.rowptr[pick.to(DEV)]
    idx = torch.repeat_interleave(starts - sub_rowptr[:-1].to(DEV), sub_counts.to(DEV)) + torch.arange(int(sub_rowptr[-1]), device=DEV)
    ci, va = g.col[idx].cpu(), g.val[idx].cpu()
    return pick, oracle_c.csr_spmm(sub_rowptr.numpy(), ci.numpy(), va.numpy(), h.float().cpu().numpy())


def spmm_properties_and_sampled_rows(g, d):
    """Size-independent properties of Y = A.H on a graph held on the device, and sampled rows (the longest, the
    shortest and random ones) against the fp64-accumulating oracle; only the sampled rows leave the device."""
    m, k = g.shape
    a = ops.CsrMatrix(g.rowptr, g.col, g.val, g.shape)
    at = ops.CsrMatrix(g.rowptr_t, g.col_t, g.val_t, (k, m))
    print(g.degree_stats(), "long rows", a.n_long_rows, "segments", a.n_segments, flush=True)
    h = S.normal_features(k, d, DEV, seed=1)
    gm = S.normal_features(m, d, DEV, seed=2)
    y = ops.spmm(a, h)
    # A.1 = row sums
    ones = torch.ones(k, 4, device=DEV)
    csum = torch.cat([torch.zeros(1, dtype=torch.float64, device=DEV), torch.cumsum(g.val.double(), 0)])  # fp64 prefix sums
    rowsum = csum[g.rowptr[1:]] - csum[g.rowptr[:-1]]
    assert rel_err(ops.spmm(a, ones)[:, 0], rowsum) <= FP32_TOL
    del csum, ones
    # adjoint identity <A.H, G> = <H, A^T.G>
    lhs = (y.double() * gm.double()).sum().item()
    rhs = (h.double() * ops.spmm(at, gm).double()).sum().item()
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), (y.double().norm() * gm.double().norm()).item() * 1e-3)
    # linearity
    y2 = ops.spmm(a, 2.0 * h + gm[:k] if m >= k else 2.0 * h)
    if m >= k:
        assert rel_err(y2, 2.0 * y.double() + ops.spmm(a, gm[:k].contiguous()).double()) <= FP32_TOL
    else:
        assert rel_err(y2, 2.0 * y.double()) <= FP32_TOL
    del y2
    # bit reproducibility
    assert torch.equal(y, ops.spmm(a, h))
    pick, ref = oracle_rows_of_spmm(g, h)
    assert rel_err(y[pick.to(DEV)].cpu(), ref) <= FP32_TOL


@pytest.mark.parametrize("scale", [0.1, 1.0])
def test_config3_properties_and_sampled_rows(scale):
    """The 2.45 M-node power-law configuration (full size and a tenth of it): size-independent
    properties of the SpMM and a comparison of sampled rows against the fp64-accumulating oracle."""
    say("config 3 at scale %g: properties" % scale)
    spmm_properties_and_sampled_rows(S.config3_graph(DEV, seed=0, scale=scale), 128)


def test_config5_full_size_bf16_spmm_properties_and_sampled_rows():
    """The bf16-storage configuration at full size: the 2.45 M-node graph, 256 features held as bf16, fp32 accumulation."""
    say("config 5 at full size: bf16 SpMM, D=256")
    g = S.config3_graph(DEV, seed=0, scale=1.0)
    m, k = g.shape
    a = ops.CsrMatrix(g.rowptr, g.col, g.val, g.shape)
    h = S.normal_features(k, 256, DEV, seed=1).to(torch.bfloat16)
    y = ops.spmm(a, h)
    assert y.dtype == torch.bfloat16 and torch.equal(y, ops.spmm(a, h))
    # sampled rows: fp32 arithmetic on the bf16-rounded inputs, one rounding of the result (2^-9 relative per element)
    pick, ref = oracle_rows_of_spmm(g, h)
    got = y[pick.to(DEV)].float().cpu()
    assert rel_err(got, ref) <= 2.0 ** -8
    # A.1 = row sums (ones are exact in bf16; the sums are rounded once)
    csum = torch.cat([torch.zeros(1, dtype=torch.float64, device=DEV), torch.cumsum(g.val.double(), 0)])
    rowsum = csum[g.rowptr[1:]] - csum[g.rowptr[:-1]]
    ones = torch.ones(k, 8, device=DEV, dtype=torch.bfloat16)
    assert rel_err(ops.spmm(a, ones)[:, 0].float(), rowsum) <= 2.0 ** -8
    # scaling by a power of two is exact in every step: Y(4 H) == 4 Y(H) bit for bit
    assert torch.equal(ops.spmm(a, 4.0 * h), 4.0 * y)


@pytest.mark.parametrize("d", [602, 128])
def test_config2_full_size_properties_and_sampled_rows(d):
    """The SpMM-only configuration at full size: R-MAT graph with 232,965 nodes and about 114.6 M entries."""
    say("config 2 at full size, D=%d: properties" % d)
    spmm_properties_and_sampled_rows(S.config2_graph(DEV, seed=0), d)


def test_config4_full_size_block_properties_and_sampled_rows():
    """One rank's block of the 2 x 2 x 2 grid at its real shape: 4,194,304 x 4,194,304, about 64 M entries, D = 64."""
    say("config 4 block at full size, D=64: properties")
    spmm_properties_and_sampled_rows(S.config4_block(DEV, seed=0), 64)


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_fused_adamw_matches_torch_and_oracle(n):
    say("fused AdamW n=%d" % n)
    from plexus_amd.optim import AdamW

    gen = torch.Generator().manual_seed(n)
    p0 = torch.randn(n, generator=gen)
    grads = [torch.randn(n, generator=gen) * (10.0 ** (i - 2)) for i in range(5)]
    for wd in (0.0, 0.01):
        p = p0.clone().to(DEV).requires_grad_()
        opt = AdamW([p], lr=3e-3, weight_decay=wd)
        ref = p0.clone().double().requires_grad_()
        ropt = torch.optim.AdamW([ref], lr=3e-3, weight_decay=wd)
        mine = [p0.clone().double()]
        state = {}
        for g in grads:
            p.grad = g.to(DEV)
            opt.step()
            ref.grad = g.double()
            ropt.step()
            po.adamw_step(mine, [g.double()], state, lr=3e-3, weight_decay=wd)
        assert rel_err(p, ref) <= FP32_TOL
        assert rel_err(p, mine[0]) <= FP32_TOL


def test_scaled_config2_rmat_spmm_wide_and_narrow():
    """SpMM-only configuration (R-MAT 0.57/0.19/0.19/0.05) at 1/50 scale, widths 602 and 128."""
    say("config 2 at 1/50 scale, D=602 and D=128")
    g = S.config2_graph(DEV, seed=0, scale=0.02)
    n = g.shape[0]
    a = ops.CsrMatrix(g.rowptr, g.col, g.val, g.shape)
    print(g.degree_stats(), "long rows", a.n_long_rows, flush=True)
    rp, ci, va = g.rowptr.cpu().numpy(), g.col.cpu().numpy(), g.val.cpu().numpy()
    for d in (602, 128):
        h = S.normal_features(n, d, DEV, seed=d)
        y = ops.spmm(a, h)
        ref = oracle_c.csr_spmm(rp, ci, va, h.cpu().numpy())
        assert rel_err(y, ref) <= FP32_TOL
        ref_t = po.spmm(torch.sparse_csr_tensor(g.rowptr.cpu(), g.col.cpu(), g.val.cpu(), size=g.shape), h.cpu())
        assert rel_err(y, ref_t) <= FP32_TOL


def test_scaled_config4_rank_block_layers():
    """One rank's block of a 2x2x2 grid at 1/64 scale: rectangular CSR block and its transpose, a
    feature slab that is a column slice of a wider matrix (ld != D), three layers fwd+bwd, no collectives."""
    say("config 4 block at 1/64 scale")
    from plexus_amd.gcn_conv import GCNConv

    g = S.config4_block(DEV, seed=0, scale=1.0 / 64)
    m, k = g.shape
    assert m == k  # rows [0, N/2) x cols [0, N/2) of a doubly permuted matrix: not symmetric
    a = ops.CsrMatrix(g.rowptr, g.col, g.val, g.shape)
    at = ops.CsrMatrix(g.rowptr_t, g.col_t, g.val_t, (k, m))
    a_cpu = torch.sparse_csr_tensor(g.rowptr.cpu(), g.col.cpu(), g.val.cpu(), size=g.shape)
    at_cpu = torch.sparse_csr_tensor(g.rowptr_t.cpu(), g.col_t.cpu(), g.val_t.cpu(), size=(k, m))
    assert not torch.equal(g.rowptr, g.rowptr_t)
    gen = torch.Generator().manual_seed(0)
    wide = torch.randn(k, 128, generator=gen)
    slab = wide[:, 64:128]  # this rank's half of the feature columns
    dims = [64, 64, 64, 24]
    ws = [po.kaiming_uniform_weight(dims[i], dims[i + 1], gen) for i in range(3)]
    go = torch.randn(m, dims[-1], generator=gen)

    # oracle: three layers with ReLU between, backward by the reference's formulas
    layers = [GCNConv(dims[i], dims[i + 1], i + 1, weight=ws[i], fuse_relu=(i < 2)) for i in range(3)]
    x = wide.to(DEV)[:, 64:128].requires_grad_()  # non-contiguous view: row pitch 128, width 64
    hcur = x
    acts = []
    for layer in layers:
        hcur = layer(hcur, [(a, at)])
        acts.append(hcur)
    hcur.backward(go.to(DEV))

    # oracle: three layers with ReLU between, backward by the reference's formulas.  The ReLU masks of
    # the backward pass are pinned to the ones the GPU forward produced: a pre-activation within rounding
    # of zero can take either sign in two fp32 summation orders (the forward outputs are compared on
    # their own, and the masks may differ in a handful of such elements only).
    net = po.OracleNet(ws, dims)
    out_ref = net.forward(slab.contiguous(), [(a_cpu, at_cpu)])
    net64 = po.OracleNet([w.double() for w in ws], dims)
    out64 = net64.forward(slab.contiguous().double(), [(a_cpu.double(), at_cpu.double())])
    masks = [(acts[0] > 0).cpu(), (acts[1] > 0).cpu(), None]
    for i in range(2):
        flips = int((masks[i] != (net64._saved[i][3] > 0)).sum())
        print("layer %d: %d ReLU mask elements differ from the fp64 oracle" % (i, flips), flush=True)
        assert flips <= 4
        assert rel_err(acts[i], torch.relu(net._saved[i][3])) <= FP32_TOL
    gx_ref, gws_ref = net.backward(go, masks)
    gx64, gws64 = net64.backward(go.double(), masks)
    assert_parity(hcur, out_ref, out64, what="OUT")
    assert_parity(x.grad, gx_ref.reshape(k, 64), gx64.reshape(k, 64), what="grad_x")
    for i, layer in enumerate(layers):
        assert_parity(layer.weight.grad, gws_ref[i], gws64[i], what="grad_w[%d]" % i)


# ---------------------------------------------------------------------------------------------------
# bf16 storage with fp32 accumulation; fused dropout
# ---------------------------------------------------------------------------------------------------
def bf(t):
    return t.to(torch.bfloat16)


BF16_GEMM_SHAPES = [(1, 1, 1), (5, 3, 2), (127, 16, 33), (128, 32, 64), (300, 47, 256), (1000, 256, 256), (513, 128, 100),
                    (260, 7, 16), (150, 256, 264), (64, 130, 70)]


def test_cast_bf16():
    say("cast fp32 -> bf16, plain and transposed")
    gen = torch.Generator().manual_seed(0)
    for shape in [(1, 1), (33, 7), (256, 256), (100, 47), (5, 300)]:
        x = torch.randn(*shape, generator=gen)
        assert torch.equal(ops.cast_bf16(x.to(DEV)).cpu(), bf(x))
        assert torch.equal(ops.cast_bf16(x.to(DEV), transpose=True).cpu(), bf(x.t().contiguous()))


@pytest.mark.parametrize("m,n,k", BF16_GEMM_SHAPES)
def test_gemm_nt_bf16(m, n, k):
    say("gemm_nt_bf16 %dx%dx%d" % (m, n, k))
    gen = torch.Generator().manual_seed(m + 7 * n + k)
    a = bf(torch.randn(m, k, generator=gen))
    b = bf(torch.randn(n, k, generator=gen))
    ref = oracle_c.gemm(a.float().numpy(), b.float().numpy(), tb=True)  # fp64 accumulation of the bf16 inputs
    c = ops.gemm_nt_bf16(a.to(DEV), b.to(DEV)).float().cpu()
    assert rel_err(c, ref) <= 2.0 ** -8  # fp32 accumulation: only the final rounding to bf16 is left
    # ReLU + mask + alpha
    act = bf(torch.relu(torch.randn(m, k, generator=gen)))
    cm = ops.gemm_nt_bf16(a.to(DEV), b.to(DEV), mask=act.to(DEV), alpha=2.0, relu=True).float().cpu()
    refm = np.maximum(2.0 * oracle_c.gemm((a.float() * (act > 0)).numpy(), b.float().numpy(), tb=True), 0)
    assert rel_err(cm, refm) <= 2.0 ** -8 and (cm >= 0).all()


@pytest.mark.parametrize("m,n,k", [(300, 256, 64), (1000, 47, 128), (129, 100, 256), (64, 8, 8)])
@pytest.mark.parametrize("p", [0.5, 0.25])
def test_gemm_nt_bf16_dropout_mask_is_the_oracles(m, n, k, p):
    say("fused dropout %dx%dx%d p=%g" % (m, n, k, p))
    gen = torch.Generator().manual_seed(m + n)
    a = bf(torch.rand(m, k, generator=gen) + 0.1)  # positive products: every kept element is > 0
    b = bf(torch.rand(n, k, generator=gen) + 0.1)
    seed, offset = 1234567890123, 77
    c = ops.gemm_nt_bf16(a.to(DEV), b.to(DEV), relu=True, dropout_p=p, seed=seed, offset=offset).float().cpu()
    keep = torch.from_numpy(po.dropout_keep_mask(m * n, seed, offset, p).reshape(m, n))
    assert torch.equal(c > 0, keep)  # bit-exact mask
    assert abs(keep.float().mean().item() - (1 - p)) < 0.02
    ref = oracle_c.gemm(a.float().numpy(), b.float().numpy(), tb=True) * keep.numpy() / (1 - p)
    assert rel_err(c, ref) <= 2.0 ** -8
    # another offset gives another mask
    c2 = ops.gemm_nt_bf16(a.to(DEV), b.to(DEV), relu=True, dropout_p=p, seed=seed, offset=offset + 1).float().cpu()
    assert not torch.equal(c2 > 0, keep)


# the last three: more than one 128 x 128 tile and at most 256 x 256, which one workgroup per stretch of rows holds whole
@pytest.mark.parametrize("m,n,k", BF16_GEMM_SHAPES + [(70000, 256, 256), (40000, 47, 256), (70001, 256, 136), (33333, 200, 256), (20011, 136, 248)])
def test_gemm_tn_bf16(m, n, k):
    say("gemm_tn_bf16 %dx%dx%d" % (m, n, k))
    gen = torch.Generator().manual_seed(m * 5 + n + k)
    a = bf(torch.randn(m, k, generator=gen))
    g = bf(torch.randn(m, n, generator=gen))
    c = ops.gemm_tn_bf16(a.to(DEV), g.to(DEV)).cpu()
    assert c.shape == (k, n) and c.dtype == torch.float32
    ref = oracle_c.gemm(a.float().numpy(), g.float().numpy(), ta=True)
    err = rel_err(c, ref)
    print("rel err %.2e" % err, flush=True)
    assert err <= FP32_TOL  # bf16 products are exact in fp32; only the fp32 summation order differs
    act = bf(torch.relu(torch.randn(m, n, generator=gen)))
    cm = ops.gemm_tn_bf16(a.to(DEV), g.to(DEV), mask=act.to(DEV), alpha=2.0).cpu()
    assert rel_err(cm, 2.0 * oracle_c.gemm(a.float().numpy(), (g.float() * (act > 0)).numpy(), ta=True)) <= FP32_TOL
    assert torch.equal(c, ops.gemm_tn_bf16(a.to(DEV), g.to(DEV)).cpu())  # bit-reproducible


@pytest.mark.parametrize("m,n,k,kin", [(40000, 256, 256, 256), (3001, 128, 256, 200), (777, 64, 96, 64), (20011, 256, 136, 248),
                                         (33, 8, 8, 16)])
def test_bf16_mask_as_bits(m, n, k, kin):
    """The forward product writes the sign bits of its bf16 result; the two backward products read the mask in that form
    and give the same bits as with the bf16 mask.  A mask of all ones in the bits, against the real mask in the values,
    shows which of the two a kernel read."""
    say("bf16 sign bits M=%d N=%d K=%d, backward into %d" % (m, n, k, kin))
    gen = torch.Generator().manual_seed(m + n + k)
    a = bf(torch.randn(m, k, generator=gen)).to(DEV)
    wt = bf(torch.randn(n, k, generator=gen) * 0.1).to(DEV)
    c, bits = ops.gemm_nt_bf16(a, wt, relu=True, want_bits=True)
    assert torch.equal(c, ops.gemm_nt_bf16(a, wt, relu=True))
    assert torch.equal(bits.cpu(), _pack_bits(c.float().cpu()))
    cd, bits_d = ops.gemm_nt_bf16(a, wt, relu=True, dropout_p=0.5, seed=99, offset=3, want_bits=True)
    assert torch.equal(cd, ops.gemm_nt_bf16(a, wt, relu=True, dropout_p=0.5, seed=99, offset=3))
    assert torch.equal(bits_d.cpu(), _pack_bits(cd.float().cpu()))
    assert not torch.equal(bits_d, bits)
    # GRAD_AGG = (G * mask) . W^T with W stored [kin x n]; GRAD_W = AGG^T . (G * mask)
    g = bf(torch.randn(m, n, generator=gen)).to(DEV)
    w = bf(torch.randn(kin, n, generator=gen) * 0.1).to(DEV)
    agg = bf(torch.randn(m, kin, generator=gen)).to(DEV)
    ones = torch.full((m, bits.stride(0) if m > 1 else 4), -1, dtype=torch.int32, device=DEV)[:, :bits.shape[1]]  # the pitch of the real ones
    by_values = ops.gemm_nt_bf16(g, w, mask=cd, alpha=2.0)
    assert torch.equal(ops.gemm_nt_bf16(g, w, mask=cd, alpha=2.0, mask_bits=bits_d), by_values)
    read_bits = ops.gemm_nt_bf16(g, w, mask=cd, alpha=2.0, mask_bits=ones)
    assert torch.equal(read_bits, ops.gemm_nt_bf16(g, w, alpha=2.0))  # N = kin and K = n are at most 256: this kernel reads the bits
    assert not torch.equal(read_bits, by_values)
    tn_values = ops.gemm_tn_bf16(agg, g, mask=cd, alpha=0.5)
    assert torch.equal(ops.gemm_tn_bf16(agg, g, mask=cd, alpha=0.5, mask_bits=bits_d), tn_values)
    whole_tile = (kin > 128 or n > 128) and m >= 1024  # more than one 128 x 128 tile and more than one stretch of rows
    tn_ones = ops.gemm_tn_bf16(agg, g, mask=cd, alpha=0.5, mask_bits=ones)
    assert torch.equal(tn_ones, ops.gemm_tn_bf16(agg, g, alpha=0.5) if whole_tile else tn_values)
    with pytest.raises(ValueError):
        ops.gemm_nt_bf16(g, w, mask_bits=bits_d)  # bits come beside the bf16 mask they stand for
    ref = oracle_c.gemm(agg.float().cpu().numpy(), (g.float() * (cd > 0)).cpu().numpy(), ta=True) * 0.5
    assert rel_err(tn_values.cpu(), ref) <= FP32_TOL


def test_bf16_sign_bits_are_refused_for_shapes_without_them():
    say("bf16 sign bits beyond 256 columns")
    a = bf(torch.randn(100, 64)).to(DEV)
    wt = bf(torch.randn(264, 64)).to(DEV)
    assert not ops.bf16_bits_supported(264, 64)
    with pytest.raises(RuntimeError, match="sign bits"):
        ops.gemm_nt_bf16(a, wt, relu=True, want_bits=True)


@pytest.mark.parametrize("m,c", [(10, 7), (1000, 47), (257, 100), (50, 1000), (1031, 41), (333, 64)])
def test_softmax_xent_bf16(m, c):
    say("softmax_xent bf16 %dx%d" % (m, c))
    gen = torch.Generator().manual_seed(m + c)
    logits = bf(torch.randn(m, c, generator=gen) * 3)
    y = torch.randint(0, c, (m,), generator=gen)
    loss, dl = ops.softmax_xent(logits.to(DEV), y.to(DEV), m, c)
    assert dl.dtype == torch.bfloat16
    closs, cgrad = oracle_c.softmax_xent(logits.float().numpy(), y.numpy(), m, c)
    assert abs(loss.item() - closs) <= FP32_TOL * abs(closs)  # the loss itself is fp32 math on the bf16 logits
    assert rel_err(dl.float().cpu(), cgrad) <= 2.0 ** -8


@pytest.mark.parametrize("n", [10007, 300 * 1024])  # scalar kernel; four-element vector kernel
def test_adamw_bf16_gradient_and_shadow(n):
    say("AdamW with bf16 gradient and bf16 shadow, n=%d" % n)
    from plexus_amd.optim import AdamW

    gen = torch.Generator().manual_seed(3)
    master0 = torch.randn(n, generator=gen)
    master = master0.clone().to(DEV)
    shadow = bf(master).clone().requires_grad_()
    opt = AdamW([master], lr=3e-3, weight_decay=0.0, shadows=[(master, shadow)])
    mine = [master0.clone().double()]
    state = {}
    for i in range(4):
        g = bf(torch.randn(n, generator=gen))
        shadow.grad = g.to(DEV)
        opt.step()
        po.adamw_step(mine, [g.double()], state, lr=3e-3)
        opt.zero_grad()
        assert shadow.grad is None
    assert rel_err(master, mine[0]) <= FP32_TOL
    assert torch.equal(shadow.detach().cpu(), bf(master.cpu()))


def test_bf16_three_layer_network_with_dropout():
    """Wide-hidden bf16 configuration at 1/100 scale: 256-256-256-47, dropout 0.5 after each ReLU,
    forward, loss and backward against the bf16-storage oracle."""
    say("config 5 at 1/100 scale: bf16 storage, dropout 0.5")
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.train import Net

    g = S.config3_graph("cpu", seed=1, scale=0.01)
    n = g.shape[0]
    dims = [256, 256, 256, 47]
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, dims[0], generator=gen)
    y = torch.randint(0, 47, (n,), generator=gen)
    ws = S.glorot_weights(dims, seed=2)
    seed = 42

    model = Net(3, dims[0], dims[1], dims[-1], weights=ws, fuse_relu=True, dropout=0.5, dropout_seed=seed)
    model.train()
    offsets = [layer.next_dropout_offset() for layer in model.layers]
    shards = [(to_dev(g), to_dev(g, True))]
    xd = bf(x).to(DEV).requires_grad_()
    logits = model(xd, shards)
    loss = parallel_cross_entropy(logits, y.to(DEV), 3, n, 47)
    loss.backward()

    net = po.OracleNetBf16(ws, dims, dropout_p=0.5, seed=seed)
    ref_logits = net.forward(x, [(g.torch_csr(), g.torch_csr(True))], offsets)
    ref_loss, sm, oh = po.cross_entropy_forward(ref_logits, y, n, 47)
    gl = po.cross_entropy_backward(sm, oh.float(), n)
    gx_ref, gws_ref = net.backward(gl)

    assert logits.dtype == torch.bfloat16 and xd.grad.dtype == torch.bfloat16
    assert rel_err(logits.float(), ref_logits) <= BF16_TOL
    assert abs(loss.item() - ref_loss.item()) <= BF16_TOL * abs(ref_loss.item())
    assert rel_err(xd.grad.float(), gx_ref.reshape(n, dims[0])) <= BF16_TOL
    for layer, gw in zip(model.layers, gws_ref):
        assert layer.weight.grad.dtype == torch.float32
        assert rel_err(layer.weight.grad, gw) <= BF16_TOL
    # the narrowing last layer computed as A.(H.W): same result within the bf16 bar
    model_tf = Net(3, dims[0], dims[1], dims[-1], weights=ws, fuse_relu=True, dropout=0.5, dropout_seed=seed, association="auto")
    assert model_tf.layers[2].transform_first and not model_tf.layers[0].transform_first
    model_tf.train()
    x_tf = bf(x).to(DEV).requires_grad_()
    logits_tf = model_tf(x_tf, shards)
    parallel_cross_entropy(logits_tf, y.to(DEV), 3, n, 47).backward()
    assert rel_err(logits_tf.float(), ref_logits) <= BF16_TOL
    assert rel_err(x_tf.grad.float(), gx_ref.reshape(n, dims[0])) <= BF16_TOL
    for layer, gw in zip(model_tf.layers, gws_ref):
        assert rel_err(layer.weight.grad, gw) <= BF16_TOL
    # eval mode: no dropout, deterministic
    model.eval()
    e1 = model(xd.detach(), shards)
    e2 = model(xd.detach(), shards)
    assert torch.equal(e1, e2)
    net0 = po.OracleNetBf16(ws, dims, dropout_p=0.0)
    assert rel_err(e1.float(), net0.forward(x, [(g.torch_csr(), g.torch_csr(True))])) <= BF16_TOL


def test_internal_timers_use_the_reference_names():
    say("timers")
    import plexus_amd
    from plexus_amd.gcn_conv import GCNConv
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.utils.timers import get_timers

    plexus_amd.init(enable_internal_timers=True)
    try:
        get_timers().reset()
        g = graph_small(n=300, pairs=2000, seed=1)
        layer = GCNConv(12, 5, 0)
        x = torch.randn(300 * 12, device=DEV, requires_grad=True)
        y = torch.randint(0, 5, (300,), device=DEV)
        loss = parallel_cross_entropy(layer(x, [(to_dev(g), to_dev(g, True))]), y, 1, 300, 5)
        loss.backward()
        times = get_timers().get_times()
        for name in ["gcn conv fwd", "AGG = A * H", "OUT = AGG * W", "gcn conv bwd", "GRAD_W = AGG.T * GRAD_OUT",
                     "GRAD_AGG = GRAD_OUT * W.T", "GRAD_H = A.T * GRAD_AGG", "cross entropy fwd", "cross entropy bwd"]:
            assert name in times and times[name] >= 0.0
    finally:
        plexus_amd.init()
        get_timers().reset()


@pytest.mark.parametrize("din,dout,relu", [(128, 47, False), (100, 16, True), (64, 64, True), (33, 5, False)])
def test_transform_first_association_matches_reference_order(din, dout, relu):
    """A.(H.W) instead of (A.H).W is the same matrix; checked against the reference-order oracle."""
    say("transform-first layer %d->%d relu=%s" % (din, dout, relu))
    from plexus_amd.gcn_conv import GCNConv

    n = 1500
    g = S.build_graph(n, "chunglu", 20000, seed=7, device="cpu")
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(n, din, generator=gen)
    w = po.kaiming_uniform_weight(din, dout, gen)
    go = torch.randn(n, dout, generator=gen)
    outs, gxs, gws = [], [], []
    for dt in (torch.float32, torch.float64):
        a, at = g.torch_csr().to(dt), g.torch_csr(True).to(dt)
        out_ref, agg_ref = po.gcn_conv_forward(x.to(dt), a, w.to(dt), (n, din), (din, dout))
        outs.append(torch.relu(out_ref) if relu else out_ref)
    layer = GCNConv(din, dout, 1, weight=w, fuse_relu=relu, association="transform_first")
    assert layer.transform_first
    xd = x.to(DEV).requires_grad_()
    out = layer(xd, [(to_dev(g), to_dev(g, True))])
    out.backward(go.to(DEV))
    assert_parity(out, outs[0], outs[1], what="OUT")
    mask = (out > 0).cpu() if relu else None  # pin the ReLU mask to the device's (sign of values within rounding of 0)
    for dt in (torch.float32, torch.float64):
        a, at = g.torch_csr().to(dt), g.torch_csr(True).to(dt)
        _, agg_ref = po.gcn_conv_forward(x.to(dt), a, w.to(dt), (n, din), (din, dout))
        gm = go.to(dt) * mask.to(dt) if relu else go.to(dt)
        gx, gw = po.gcn_conv_backward(gm, agg_ref, w.to(dt), at, (din, dout))
        gxs.append(gx)
        gws.append(gw)
    assert_parity(xd.grad, gxs[0], gxs[1], what="grad_x")
    assert_parity(layer.weight.grad, gws[0], gws[1], what="grad_w")
    # "auto" picks it exactly when the gathered rows get shorter in 128-byte lines
    assert GCNConv(128, 47, 2, association="auto").transform_first
    assert GCNConv(1433, 16, 0, association="auto").transform_first
    assert not GCNConv(100, 128, 0, association="auto").transform_first
    assert not GCNConv(128, 128, 1, association="auto").transform_first
    assert not GCNConv(128, 47, 2).transform_first


def test_config1_ten_epochs_with_auto_association():
    say("config 1, 10 epochs, association=auto")
    from plexus_amd.train import Net, make_optimizer, run_epochs

    g, x, y, dims = S.config1(device="cpu", seed=0)
    weights = S.glorot_weights(dims, seed=0)
    n = g.shape[0]
    ref64, x64, w64 = po.train_epochs(x.double(), [w.double() for w in weights], dims,
                                      [(g.torch_csr().double(), g.torch_csr(True).double())], y, n, 7, epochs=10)
    model = Net(2, dims[0], dims[1], dims[2], weights=weights, association="auto")
    assert model.layers[0].transform_first and not model.layers[1].transform_first  # 16 -> 7 stays inside one line
    feats = x.reshape(-1).to(DEV).requires_grad_()
    opt = make_optimizer(model, feats)
    shards = [(g.torch_csr().to(DEV), g.torch_csr(True).to(DEV))]
    losses = run_epochs(model, opt, feats, shards, y.to(DEV), n, 7, 10)
    for l, r64 in zip(losses, ref64):
        assert abs(l - r64) <= FP32_TOL * abs(r64)


def test_spmm_from_a_line_aligned_copy_of_h_gives_the_same_bits():
    say("spmm: staging of H into line-aligned rows")
    from plexus_amd import _lib

    g = S.build_graph(3000, "chunglu", 40000, seed=9, device="cpu", gamma=2.1)
    per_row_of_h = g.nnz / 3000  # about 27: enough to repay the copy of 188-byte rows, not that of 2,408-byte rows
    assert 15 < per_row_of_h < 60
    a = to_dev(g, seg_len=128)
    lib = _lib.load()
    for d, staged in ((47, True), (602, False), (100, False), (128, False), (24, True)):
        seg_only = a.n_segments * ((d + 3) // 4 * 4) * 4
        need = int(lib.plx_spmm_workspace_bytes(a._plan, d))
        assert (need > seg_only) == staged, (d, need, seg_only)
        h = torch.randn(3000, d, generator=torch.Generator().manual_seed(d)).to(DEV)
        y = ops.spmm(a, h)  # whole matrix: gathers from the copy when the workspace has room for it
        y_rows = ops.chunked_spmm(a, h, max_rows_per_chunk=1100)  # row ranges never stage
        assert torch.equal(y, y_rows)
        assert rel_err(y.cpu(), oracle_spmm64(g, h.cpu())) <= FP32_TOL
        # an operand that is already line-aligned is used where it lies
        hp = torch.zeros(3000, (d + 31) // 32 * 32, device=DEV)
        hp[:, :d] = h
        assert torch.equal(ops.spmm(a, hp[:, :d]), y)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_spmm_in_column_slices_agrees_bit_for_bit_with_its_one_pass_form(dtype):
    """Products of a sliced shape: passes over 256-byte column slices of H (in place when its rows lie on 128-byte lines,
    else from a staged copy), and the one-pass kernel that sums in the same order (row ranges, operands that can be
    neither sliced in place nor copied).  All of them must give the same bits, and the oracle's numbers."""
    say("spmm in column slices, %s" % dtype)
    from plexus_amd import _lib

    lib = _lib.load()
    g = S.build_graph(3000, "chunglu", 40000, seed=5, device="cpu", gamma=2.1)
    tol = FP32_TOL if dtype == torch.float32 else 2.0 ** -8
    per16 = 4 if dtype == torch.float32 else 8
    widths = [128, 602, 130, 72, 256, 1433] if dtype == torch.float32 else [256, 200, 136, 602]
    for seg_len in (64, 1024):
        a = to_dev(g, seg_len=seg_len)
        plain = to_dev(g, seg_len=seg_len)
        plain.set_slicing(-1)
        a.set_slicing(1)
        assert a.n_long_rows > 0
        for d in widths:
            h_host = torch.randn(3000, d, generator=torch.Generator().manual_seed(d)).to(dtype)
            h = h_host.to(DEV)
            y = ops.spmm(a, h)  # whole matrix: sliced in place (rows on lines, whole 16-byte units) or from a copy
            assert rel_err(y.float().cpu(), oracle_spmm64(g, h_host.float())) <= tol
            # row ranges never slice: one pass with the same four chains per sum
            assert torch.equal(ops.chunked_spmm(a, h, max_rows_per_chunk=700), y), (d, seg_len)
            # an operand off the lines and no room to copy it (the entry point without a workspace): one pass again
            if dtype == torch.float32 and a.n_segments * ((d + 3) // 4) * 16 <= (32 << 20):
                y2 = torch.full((3000, d), float("nan"), device=DEV)
                flat = torch.zeros(3000 * d + 1, device=DEV)
                h_off = flat[1:].view(3000, d)
                h_off.copy_(h)
                _lib.check(lib.plx_spmm_csr_f32_static(a._plan, a.val.data_ptr(), h_off.data_ptr(), d, d, y2.data_ptr(), d,
                                                       torch.cuda.current_stream().cuda_stream), "plx_spmm_csr_f32_static")
                assert torch.equal(y2, y), (d, seg_len)
            # H and Y as column slabs of wider matrices; Y rows off 16-byte boundaries
            wide_h = torch.zeros(3000, d + 32 * per16, device=DEV, dtype=dtype)
            wide_h[:, 32 * per16 // 2: 32 * per16 // 2 + d] = h
            wide_y = torch.zeros(3000, d + 3, device=DEV, dtype=dtype)
            ops.spmm(a, wide_h[:, 32 * per16 // 2: 32 * per16 // 2 + d], out=wide_y[:, 1:1 + d])
            assert torch.equal(wide_y[:, 1:1 + d], y) and (wide_y[:, 0] == 0).all() and (wide_y[:, 1 + d:] == 0).all(), (d, seg_len)
            # the unsliced product differs in summation order only
            assert rel_err(ops.spmm(plain, h).float(), y.float()) <= (1e-6 if dtype == torch.float32 else 2.0 ** -7)
    # the rule itself: this small matrix is not sliced unless told to, the 233 K-row benchmark matrix would be
    auto = to_dev(g)
    h = torch.randn(3000, 602, generator=torch.Generator().manual_seed(1)).to(DEV)
    assert torch.equal(ops.spmm(auto, h), ops.spmm(plain, h))


def _hub_matrix(seed, n=3000, pairs=40000, seg_len=16):
    g = S.build_graph(n, "chunglu", pairs, seed=seed, device="cpu", gamma=2.1)
    a = to_dev(g, seg_len=seg_len)
    assert a.n_hub_rows == 0  # too small for the library to build the tables by itself
    a.build_hub()
    return g, a


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d", [4, 64, 100, 128, 260, 512])
def test_spmm_hub_pass_matches_the_oracle_and_keeps_its_bits(d, dtype):
    say("spmm hub pass D=%d %s" % (d, dtype))
    g, a = _hub_matrix(seed=31)
    # split rows of more than 16 * seg_len entries take several parts; the longest rows all become hub rows
    assert a.n_hub_rows == a.n_long_rows > 100 and g.degree_stats()["max_row_nnz"] > 16 * 16
    assert a.hub_entries > g.nnz // 3
    h32 = torch.randn(3000, d, generator=torch.Generator().manual_seed(d))
    h = h32.to(dtype).to(DEV)
    ref = oracle_spmm64(g, h.float().cpu())
    tol = FP32_TOL if dtype == torch.float32 else BF16_TOL
    y = ops.spmm(a, h)
    assert rel_err(y.float().cpu(), ref) <= tol
    assert torch.equal(ops.spmm(a, h), y)  # the order of every sum is fixed by the plan
    assert torch.equal(ops.chunked_spmm(a, h, max_rows_per_chunk=700), y)  # row ranges run the same pass
    a.set_hub(-1)
    y_plain = ops.spmm(a, h)
    a.set_hub(0)
    assert rel_err(y_plain.float().cpu(), ref) <= tol
    taken = d * h.element_size() >= 256  # narrower rows do not repay the pass (this matrix has 7 entries per slot and window)
    if not taken:
        assert torch.equal(y_plain, y)
    elif dtype == torch.float32:
        assert not torch.equal(y_plain, y)  # the pass was taken: hub rows are summed in another order
        assert rel_err(y.cpu(), y_plain.cpu()) <= 2e-6
    # the rows that are not hub rows are summed as without the pass
    rows = torch.ones(3000, dtype=torch.bool)
    long_rows = torch.nonzero((g.rowptr[1:] - g.rowptr[:-1]) > 16).reshape(-1)
    rows[long_rows] = False
    assert torch.equal(y.cpu()[rows], y_plain.cpu()[rows])


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_spmm_hub_pass_on_random_shapes(seed):
    """Rectangular matrices with a few very long rows, every width class and both element types, against the fp64 oracle."""
    say("spmm hub pass, random shape %d" % seed)
    gen = torch.Generator().manual_seed(100 + seed)
    m = int(torch.randint(50, 4000, (1,), generator=gen))
    k = int(torch.randint(9, 30000, (1,), generator=gen))
    seg_len = [2, 8, 64, 256][seed % 4]
    # row lengths: mostly short, some far beyond a part (16 * seg_len), one covering every column
    lens = torch.randint(0, 6, (m,), generator=gen)
    long_rows = torch.randperm(m, generator=gen)[: max(3, m // 20)]
    lens[long_rows] = torch.randint(seg_len + 1, max(seg_len + 2, min(k, 40 * seg_len)), (long_rows.numel(),), generator=gen)
    lens[long_rows[0]] = k
    lens = lens.clamp(max=k)
    cols = [torch.randperm(k, generator=gen)[: int(n)].sort().values for n in lens]
    rowptr = torch.zeros(m + 1, dtype=torch.int64)
    rowptr[1:] = torch.cumsum(lens, 0)
    col = torch.cat(cols).to(torch.int32)
    val = torch.randn(col.numel(), generator=gen)
    a = ops.CsrMatrix(rowptr.to(torch.int32).to(DEV), col.to(DEV), val.to(DEV), (m, k), seg_len)
    a.build_hub()
    assert a.n_hub_rows > 0
    for d, dtype in ((128, torch.float32), (64, torch.float32), (388, torch.float32), (256, torch.bfloat16), (132, torch.bfloat16)):
        h = torch.randn(k, d, generator=gen).to(dtype)
        ref = oracle_c.csr_spmm(rowptr.to(torch.int32).numpy(), col.numpy(), val.numpy(), h.float().numpy())
        y = ops.spmm(a, h.to(DEV))
        assert rel_err(y.float().cpu(), ref) <= (FP32_TOL if dtype == torch.float32 else BF16_TOL), (m, k, seg_len, d, dtype)
        assert torch.equal(ops.chunked_spmm(a, h.to(DEV), max_rows_per_chunk=max(1, m // 3)), y)


def test_spmm_workspace_covers_the_hub_pass_of_either_storage_type():
    """With column slicing forced on, 128 fp32 columns (512-byte rows) are sliced and take no hub pass, while 128 bf16
    columns (256-byte rows) are not sliced and do: each storage type has its size query, and each product checks what it
    was given against its own."""
    say("spmm: slicing forced on + hub tables, D=128 in fp32 and bf16")
    from plexus_amd import _lib

    lib = _lib.load()
    g, a = _hub_matrix(seed=34)
    a.set_slicing(1)
    d = 128
    seg_bytes = a.n_segments * d * 4
    partial = 8 * 9216 * 128 * 4  # ranges x slots x columns of the partial sums of a pass
    need = int(lib.plx_spmm_workspace_bytes_bf16(a._plan, d))
    assert need >= seg_bytes + partial > int(lib.plx_spmm_workspace_bytes(a._plan, d))  # the fp32 product takes slices, no pass
    h32 = torch.randn(3000, d, generator=torch.Generator().manual_seed(7))
    ref = oracle_spmm64(g, h32.to(torch.bfloat16).float())
    # behind the workspace lies a tensor that must come back untouched
    arena = torch.zeros(need + (1 << 20), dtype=torch.uint8, device=DEV)
    arena[need:] = 0xA5
    hb = h32.to(torch.bfloat16).to(DEV)
    y = torch.empty(3000, d, dtype=torch.bfloat16, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.plx_spmm_csr_bf16(a._plan, a.val.data_ptr(), hb.data_ptr(), d, d, y.data_ptr(), d, arena.data_ptr(), need, st), "plx_spmm_csr_bf16")
    assert rel_err(y.float().cpu(), ref) <= BF16_TOL
    assert (arena[need:] == 0xA5).all()
    assert torch.equal(ops.spmm(a, hb), y)  # through the front end, which sizes its workspace with the same query
    # a workspace that holds the partial rows of the split rows only is refused, not overrun
    rc = lib.plx_spmm_csr_bf16(a._plan, a.val.data_ptr(), hb.data_ptr(), d, d, y.data_ptr(), d, arena.data_ptr(), seg_bytes, st)
    assert rc == _lib.PLX_ERR_WORKSPACE
    # the fp32 product of the same width runs in column slices and agrees with the oracle too
    yf = ops.spmm(a, h32.to(DEV))
    assert rel_err(yf.cpu(), oracle_spmm64(g, h32)) <= FP32_TOL


def test_spmm_hub_pass_in_the_wide_layout_for_bf16_rows_of_512_bytes():
    """bf16 products of 256 columns and more take the hub pass in its wide layout (256-column tiles, 18 sums per
    wavefront, 16-byte loads) once the plan has those tables; widths and operands that do not allow 16-byte loads keep
    the regular layout.  Both against the fp64 oracle, the wide one also bit-stable on repeat and in row ranges."""
    say("spmm hub pass, wide layout (bf16, D >= 256)")
    g, a = _hub_matrix(seed=36)
    regular_only = to_dev(g, seg_len=16)
    regular_only.build_hub()
    regular_only._wide_tried = True  # keeps the front end from building the wide tables for this one
    n = 3000
    for d in (256, 264, 512, 1000):
        h = torch.randn(n, d, generator=torch.Generator().manual_seed(d)).to(torch.bfloat16).to(DEV)
        ref = oracle_spmm64(g, h.float().cpu())
        y = ops.spmm(a, h)
        assert a.n_hub_rows_wide > 0 and regular_only.n_hub_rows_wide == 0
        assert rel_err(y.float().cpu(), ref) <= BF16_TOL, d
        assert torch.equal(ops.spmm(a, h), y)
        assert torch.equal(ops.chunked_spmm(a, h, max_rows_per_chunk=700), y)
        y_reg = ops.spmm(regular_only, h)
        assert rel_err(y_reg.float().cpu(), ref) <= BF16_TOL
        # fp32 sums in another order, rounded to bf16 at the end: equal but for an element in a few thousand
        assert (y != y_reg).float().mean().item() < 0.02 and rel_err(y.float(), y_reg.float()) <= 2.0 ** -7
        # rows outside the pass are summed by the row kernel either way
        rows = torch.ones(n, dtype=torch.bool)
        rows[torch.nonzero((g.rowptr[1:] - g.rowptr[:-1]) > 16).reshape(-1)] = False
        assert torch.equal(y.cpu()[rows], y_reg.cpu()[rows])
    # a width that is no multiple of 8, and a view 8 bytes into a wider matrix: the regular tables, bit for bit
    h = torch.randn(n, 260, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(DEV)
    assert torch.equal(ops.spmm(a, h), ops.spmm(regular_only, h))
    wide = torch.randn(n, 272, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).to(DEV)
    view = wide[:, 4:260]
    assert view.data_ptr() % 16 == 8
    assert torch.equal(ops.spmm(a, view), ops.spmm(regular_only, view))
    assert rel_err(ops.spmm(a, view).float().cpu(), oracle_spmm64(g, view.float().cpu().contiguous())) <= BF16_TOL
    # fp32 products never take the wide tables
    hf = torch.randn(n, 256, generator=torch.Generator().manual_seed(3)).to(DEV)
    assert torch.equal(ops.spmm(a, hf), ops.spmm(regular_only, hf))
    # switched off, the product is the row kernel's
    a.set_hub(-1)
    regular_only.set_hub(-1)
    h = torch.randn(n, 256, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).to(DEV)
    assert torch.equal(ops.spmm(a, h), ops.spmm(regular_only, h))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_chunked_product_runs_the_hub_pass_once_and_keeps_every_bit(dtype):
    """The two ways of computing a product range by range: plx_spmm_csr_rows_* (every range that holds a hub row runs the
    whole pass) and plx_spmm_csr_chunk_* (the first chunk runs it for all, later chunks add up their own hub rows from
    the partial sums it left).  Both must give the whole product's bits, also when the first chunk holds no hub row."""
    say("chunk entry points with a hub pass, %s" % dtype)
    from plexus_amd import _lib

    lib = _lib.load()
    g, a = _hub_matrix(seed=35)
    n, d = 3000, 128 if dtype == torch.float32 else 256
    h = torch.randn(n, d, generator=torch.Generator().manual_seed(3)).to(dtype).to(DEV)
    whole = ops.spmm(a, h)
    a.set_hub(-1)
    assert not torch.equal(ops.spmm(a, h), whole) or dtype == torch.bfloat16  # the pass is taken at this width
    a.set_hub(0)
    rows_fn, chunk_fn = ((lib.plx_spmm_csr_rows_f32, lib.plx_spmm_csr_chunk_f32) if dtype == torch.float32 else
                         (lib.plx_spmm_csr_rows_bf16, lib.plx_spmm_csr_chunk_bf16))
    ws, ws_bytes = a._workspace(d, dtype)
    st = torch.cuda.current_stream().cuda_stream
    hub_rows = torch.nonzero((g.rowptr[1:] - g.rowptr[:-1]) > 16).reshape(-1)
    gaps = hub_rows[1:] - hub_rows[:-1]
    i = int(torch.argmax(gaps))
    lo_free, hi_free = int(hub_rows[i]) + 1, int(hub_rows[i + 1])  # the longest run of rows without a hub row
    assert hi_free - lo_free >= 2
    # chunks in the order they are issued: the first one holds no hub row (it still runs the pass for the others); then
    # the rows before it; an empty chunk; the rows after it
    bounds = [(lo_free, hi_free), (0, lo_free), (lo_free, lo_free), (hi_free, n)]
    y_rows = torch.zeros(n, d, dtype=dtype, device=DEV)
    for lo, hi in bounds:
        _lib.check(rows_fn(a._plan, lo, hi, a.val.data_ptr(), h.data_ptr(), d, d, y_rows.data_ptr(), d, ws.data_ptr(), ws_bytes, st), "rows")
    assert torch.equal(y_rows, whole)
    y_chunk = torch.zeros(n, d, dtype=dtype, device=DEV)
    for i, (lo, hi) in enumerate(bounds):
        ws[:64] = 0  # nothing in the front of the workspace (partial rows of split rows) is carried between chunks
        _lib.check(chunk_fn(a._plan, lo, hi, int(i == 0), a.val.data_ptr(), h.data_ptr(), d, d, y_chunk.data_ptr(), d, ws.data_ptr(),
                            ws_bytes, st), "chunk")
    assert torch.equal(y_chunk, whole)
    assert rel_err(whole.float().cpu(), oracle_spmm64(g, h.float().cpu())) <= (FP32_TOL if dtype == torch.float32 else BF16_TOL)
    # a plan without hub tables: the chunk entry points are the row-range ones
    plain = to_dev(g, seg_len=16)
    y2 = torch.zeros(n, d, dtype=dtype, device=DEV)
    ws2, ws2_bytes = plain._workspace(d, dtype)
    for i, (lo, hi) in enumerate(bounds):
        _lib.check(chunk_fn(plain._plan, lo, hi, int(i == 0), plain.val.data_ptr(), h.data_ptr(), d, d, y2.data_ptr(), d,
                            ws2.data_ptr() if ws2 is not None else None, ws2_bytes, st), "chunk")
    assert torch.equal(y2, ops.spmm(plain, h))


def test_hub_tables_are_refused_for_rows_whose_columns_do_not_ascend():
    say("hub tables on a matrix with unsorted columns in a long row")
    from plexus_amd._lib import PlexusHipError

    gen = torch.Generator().manual_seed(12)
    m, k, seg_len = 50, 4000, 8
    lens = torch.full((m,), 3, dtype=torch.int64)
    lens[7] = 900
    lens[20] = 1200
    cols = [torch.randperm(k, generator=gen)[: int(n)].sort().values for n in lens]
    cols[20] = cols[20][torch.randperm(1200, generator=gen)]  # one long row in arbitrary order
    rowptr = torch.zeros(m + 1, dtype=torch.int64)
    rowptr[1:] = torch.cumsum(lens, 0)
    col = torch.cat(cols).to(torch.int32)
    val = torch.randn(col.numel(), generator=gen)
    a = ops.CsrMatrix(rowptr.to(torch.int32).to(DEV), col.to(DEV), val.to(DEV), (m, k), seg_len)
    with pytest.raises(PlexusHipError, match="do not ascend"):
        a.build_hub()
    assert a.n_hub_rows == 0
    # the product without the pass takes the columns of a row in any order
    h = torch.randn(k, 128, generator=gen)
    ref = oracle_c.csr_spmm(rowptr.to(torch.int32).numpy(), col.numpy(), val.numpy(), h.numpy())
    assert rel_err(ops.spmm(a, h.to(DEV)).cpu(), ref) <= FP32_TOL
    # sorted, the same matrix gets its tables and the same product
    order = torch.cat([rowptr[r] + torch.argsort(col[rowptr[r]:rowptr[r + 1]].to(torch.int64)) for r in range(m)])
    b = ops.CsrMatrix(rowptr.to(torch.int32).to(DEV), col[order].to(DEV), val[order].to(DEV), (m, k), seg_len)
    b.build_hub()
    assert b.n_hub_rows == 2
    assert rel_err(ops.spmm(b, h.to(DEV)).cpu(), ref) <= FP32_TOL


def test_spmm_hub_pass_is_left_out_where_the_operand_does_not_suit_it():
    say("spmm hub pass: widths and layouts it does not take")
    g, a = _hub_matrix(seed=32)
    for d in (47, 130 + 1):  # not a multiple of 4
        h = torch.randn(3000, d, generator=torch.Generator().manual_seed(d)).to(DEV)
        y = ops.spmm(a, h)
        a.set_hub(-1)
        assert torch.equal(ops.spmm(a, h), y)
        a.set_hub(0)
        assert rel_err(y.cpu(), oracle_spmm64(g, h.cpu())) <= FP32_TOL
    # a view that starts 4 bytes into a wider matrix is not 16-byte aligned
    wide = torch.randn(3000, 132, generator=torch.Generator().manual_seed(5)).to(DEV)
    h = wide[:, 1:129]
    y = ops.spmm(a, h)
    a.set_hub(-1)
    assert torch.equal(ops.spmm(a, h), y)
    a.set_hub(0)
    # a 16-byte aligned view of the same matrix is taken, and reads the view's columns only
    h = wide[:, 4:132]
    y = ops.spmm(a, h)
    assert rel_err(y.cpu(), oracle_spmm64(g, h.cpu().contiguous())) <= FP32_TOL
    a.set_hub(-1)
    assert not torch.equal(ops.spmm(a, h), y)


def test_spmm_hub_pass_on_transposes_few_columns_and_every_row_a_hub_row():
    say("spmm hub pass: small and degenerate shapes")
    # 40 rows of 300 entries over 5 columns... every row long, fewer columns than column ranges
    gen = torch.Generator().manual_seed(3)
    m, k = 40, 5
    dense = torch.randn(m, k, generator=gen)
    crow = torch.arange(0, m * k + 1, k, dtype=torch.int32)
    col = torch.arange(k, dtype=torch.int32).repeat(m)
    a = ops.CsrMatrix(crow.to(DEV), col.to(DEV), dense.reshape(-1).to(DEV), (m, k), 2)
    a.build_hub()
    assert a.n_hub_rows == m
    h = torch.randn(k, 128, generator=gen)
    y = ops.spmm(a, h.to(DEV)).cpu()
    assert rel_err(y, (dense.double() @ h.double())) <= FP32_TOL
    a.set_hub(-1)
    assert not torch.equal(ops.spmm(a, h.to(DEV)).cpu(), y)  # the pass was taken
    # the transpose of a power-law graph: columns and rows change roles, the hub rows are the popular columns
    g = S.build_graph(3000, "chunglu", 40000, seed=33, device="cpu", gamma=2.1)
    at = to_dev(g, transpose=True, seg_len=16)
    at.build_hub()
    h = torch.randn(3000, 128, generator=gen)
    y = ops.spmm(at, h.to(DEV)).cpu()
    assert rel_err(y, oracle_spmm64(g, h, transpose=True)) <= FP32_TOL
    # one row far longer than a part (several slots), repeated columns allowed by CSR are not: columns are distinct here
    k = 20000
    crow = torch.tensor([0, k, k + 3], dtype=torch.int32)
    col = torch.cat([torch.arange(k, dtype=torch.int32), torch.tensor([1, 7, 19999], dtype=torch.int32)])
    val = torch.randn(k + 3, generator=gen)
    a = ops.CsrMatrix(crow.to(DEV), col.to(DEV), val.to(DEV), (2, k), 64)
    a.build_hub()
    assert a.n_hub_rows == 1 and a.hub_entries == k
    h = torch.randn(k, 128, generator=gen)
    y = ops.spmm(a, h.to(DEV)).cpu()
    ref = torch.stack([(val[:k, None].double() * h.double()).sum(0), (val[k:, None].double() * h[[1, 7, 19999]].double()).sum(0)])
    assert rel_err(y, ref) <= FP32_TOL


def test_spmm_staging_with_bf16_rows_and_dense_reuse():
    say("spmm: staging of bf16 rows and of 2,408-byte fp32 rows under heavy reuse")
    g = S.build_graph(2000, "uniform", 0, seed=11, device="cpu", exact_pairs=100000)  # about 100 entries per column of H
    assert g.nnz / 2000 > 90
    a = to_dev(g, seg_len=64)
    d = 602
    from plexus_amd import _lib
    assert int(_lib.load().plx_spmm_workspace_bytes(a._plan, d)) >= 2000 * 2432 + a.n_segments * 604 * 4  # room for the copy
    for dtype, tol in ((torch.float32, FP32_TOL), (torch.bfloat16, 2.0 ** -8)):
        h = torch.randn(2000, d, generator=torch.Generator().manual_seed(1)).to(dtype).to(DEV)
        y = ops.spmm(a, h)  # contiguous rows: staged into line-aligned rows first
        pitch = 640  # rows that already start on 128-byte lines are gathered where they lie
        hp = torch.zeros(2000, pitch, device=DEV, dtype=dtype)
        hp[:, :d] = h
        assert torch.equal(ops.spmm(a, hp[:, :d]), y)
        assert rel_err(y.float().cpu(), oracle_spmm64(g, h.float().cpu())) <= tol


def test_row_chunked_spmm_is_bit_identical_and_hands_chunks_on():
    say("row-chunked SpMM (blocked aggregation)")
    import plexus_amd
    from plexus_amd.gcn_conv import GCNConv

    g = S.build_graph(5000, "chunglu", 60000, seed=3, device="cpu", gamma=2.1)
    a = to_dev(g, seg_len=64)
    assert a.n_long_rows > 3
    h = torch.randn(5000, 36, generator=torch.Generator().manual_seed(0)).to(DEV)
    full = ops.spmm(a, h)
    seen = []
    y = ops.chunked_spmm(a, h, max_rows_per_chunk=700, on_chunk=lambda i, rng, out: seen.append((i, rng)))
    assert torch.equal(y, full)
    assert [r for _, r in seen] == po.chunk_bounds(5000, 700)  # the reference's chunk boundaries
    assert torch.equal(ops.chunked_spmm(a, h), full)  # one chunk
    ref = po.chunked_spmm(g.torch_csr(), h.cpu(), max_rows_per_chunk=700)
    assert rel_err(y, ref) <= FP32_TOL
    # through the layer: block_aggregation gives the same output and gradients
    w = po.kaiming_uniform_weight(36, 8, torch.Generator().manual_seed(1))
    outs = []
    for blocked in (False, True):
        plexus_amd.init(block_aggregation=blocked)
        layer = GCNConv(36, 8, 1, weight=w)
        x = h.clone().requires_grad_()
        o = layer(x, [(a, to_dev(g, True))])
        o.sum().backward()
        outs.append((o.detach(), x.grad, layer.weight.grad))
    plexus_amd.init()
    for u, v in zip(*outs):
        assert torch.equal(u, v)
    # bf16 storage: the same row ranges of the bf16 product, bit for bit, alone and through the layer
    hb = h.to(torch.bfloat16)
    full_b = ops.spmm(a, hb)
    assert full_b.dtype == torch.bfloat16 and torch.equal(ops.chunked_spmm(a, hb, max_rows_per_chunk=700), full_b)
    outs = []
    for blocked in (False, True):
        plexus_amd.init(block_aggregation=blocked)
        layer = GCNConv(36, 8, 1, weight=w, fuse_relu=True)
        x = hb.clone().requires_grad_()
        o = layer(x, [(a, to_dev(g, True))])
        o.float().sum().backward()
        outs.append((o.detach(), x.grad, layer.weight.grad))
    plexus_amd.init()
    for u, v in zip(*outs):
        assert torch.equal(u, v)


def test_fp32_wrappers_reject_other_dtypes():
    say("dtype checks of the fp32 products")
    a = torch.randn(64, 16, device=DEV)
    b = torch.randn(16, 8, device=DEV)
    g = torch.randn(64, 8, device=DEV)
    for bad in (a.double(), a.half(), a.to(torch.bfloat16)):
        with pytest.raises(TypeError, match="float32"):
            ops.gemm_nn(bad, b)
        with pytest.raises(TypeError, match="float32"):
            ops.gemm_tn(bad, g)
    with pytest.raises(TypeError, match="float32"):
        ops.gemm_nn(a, b.double())
    with pytest.raises(TypeError, match="mask must be float32"):
        ops.gemm_nt(g, b, mask=g > 0)
    with pytest.raises(TypeError, match="mask must be float32"):
        ops.gemm_tn(a, g, mask=(g > 0))
    with pytest.raises(TypeError):
        ops.chunked_spmm(ops.CsrMatrix(torch.zeros(65, dtype=torch.int64, device=DEV), torch.zeros(0, dtype=torch.int64, device=DEV),
                                       torch.zeros(0, device=DEV), (64, 64)), a.double())


def test_device_csr_transpose_matches_host_construction():
    say("device CSR transpose")
    cases = [S.build_graph(3000, "chunglu", 40000, seed=1, device="cpu"),
             S.build_graph(4096, "rmat", 30000, seed=2, device="cpu", double_perm=True, block=((0, 2048), (0, 1024))),
             S.build_graph(300, "uniform", 0, seed=3, device="cpu", exact_pairs=50)]
    for g in cases:
        a = to_dev(g)
        at = ops.csr_transpose(a)
        assert at.shape == (g.shape[1], g.shape[0])
        assert torch.equal(at.rowptr.cpu().long(), g.rowptr_t)
        assert torch.equal(at.col.cpu().long(), g.col_t)
        assert torch.equal(at.val.cpu(), g.val_t)  # bit-exact: values are moved, not recomputed
        # and it is what torch builds on the host (the reference's way)
        ref = g.torch_csr().transpose(0, 1).to_sparse_csr()
        assert torch.equal(at.rowptr.cpu().long(), ref.crow_indices()) and torch.equal(at.col.cpu().long(), ref.col_indices())
        assert torch.equal(at.val.cpu(), ref.values())
    # empty matrix
    e = ops.CsrMatrix(torch.zeros(11, dtype=torch.int64, device=DEV), torch.zeros(0, dtype=torch.int64, device=DEV),
                      torch.zeros(0, device=DEV), (10, 7))
    et = ops.csr_transpose(e)
    assert et.shape == (7, 10) and et.nnz == 0 and (et.rowptr == 0).all()


def test_device_block_csr_from_edge_list_matches_loader_sequence():
    say("device COO block -> CSR pair")
    gen = torch.Generator().manual_seed(0)
    n = 500
    ei = torch.randint(0, n, (2, 6000), generator=gen)
    ei = torch.cat([ei, ei[:, :500]], dim=1)  # 500 duplicated edges: the host path sums them
    w = torch.rand(ei.shape[1], generator=gen)
    for rr, cr in [((0, n), (0, n)), ((100, 350), (0, 250)), ((0, 10), (490, 500)), ((200, 200), (0, n))]:
        a_ref, at_ref = po.build_csr_pair(ei, w, (n, n), rr, cr)
        a, at = ops.csr_pair_from_edges(ei.to(DEV), w.to(DEV), (n, n), rr, cr)
        assert a.shape == tuple(a_ref.shape) and at.shape == tuple(at_ref.shape)
        assert torch.equal(a.rowptr.cpu().long(), a_ref.crow_indices())
        assert torch.equal(a.col.cpu().long(), a_ref.col_indices())
        assert rel_err(a.val.cpu(), a_ref.values()) <= FP32_TOL if a.nnz else True
        assert torch.equal(at.rowptr.cpu().long(), at_ref.crow_indices())
        assert torch.equal(at.col.cpu().long(), at_ref.col_indices())
        assert rel_err(at.val.cpu(), at_ref.values()) <= FP32_TOL if a.nnz else True
    # the pair feeds the layer directly
    h = torch.randn(n, 16, generator=gen)
    a, at = ops.csr_pair_from_edges(ei.to(DEV), w.to(DEV), (n, n))
    a_ref, at_ref = po.build_csr_pair(ei, w, (n, n))
    assert rel_err(ops.spmm(a, h.to(DEV)), po.spmm(a_ref, h)) <= FP32_TOL
    assert rel_err(ops.spmm(at, h.to(DEV)), po.spmm(at_ref, h)) <= FP32_TOL


@pytest.mark.parametrize("k", [4, 5, 6, 7, 9, 33, 47, 63, 65, 100, 127])
@pytest.mark.parametrize("n", [16, 64, 128])
def test_rows_without_16_byte_alignment_give_exact_integer_products(k, n):
    """Small integers make every product exact in fp32, so a column that the shifted last vector of a row puts in the wrong
    place changes the result.  A has K columns (rows of 4 K bytes) and a base that is only 4-byte aligned."""
    say("exact integer products, K=%d N=%d, 4-byte aligned rows" % (k, n))
    gen = torch.Generator().manual_seed(100 * k + n)
    m = 1000 + k
    flat = torch.zeros(m * k + 1)
    flat[1:] = torch.randint(-3, 4, (m * k,), generator=gen).float()
    a = flat.to(DEV)[1:].view(m, k)
    assert a.data_ptr() % 16 != 0
    w = torch.randint(-3, 4, (k, n), generator=gen).float()
    ref = flat[1:].view(m, k).double() @ w.double()
    assert torch.equal(ops.gemm_nn(a, w.to(DEV)).cpu().double(), ref)
    assert torch.equal(ops.gemm_nt(a, w.t().contiguous().to(DEV)).cpu().double(), ref)


@pytest.mark.parametrize("n", [1, 3, 47, 63, 64])
@pytest.mark.parametrize("m", [16, 777, 4101])
def test_narrow_contiguous_results_leave_in_flat_runs_exactly(m, n):
    """A contiguous result of at most 64 columns whose rows are not multiples of 16 bytes is written as flat runs of 16-byte
    stores, 16 rows at a time; the last run of a short last panel ends element by element.  Integer operands: exact results,
    fp32 and bf16, and nothing written past the end of C."""
    say("flat epilogue %d x %d" % (m, n))
    gen = torch.Generator().manual_seed(m + n)
    k = 128
    a = torch.randint(-1, 2, (m, k), generator=gen).float()
    w = torch.randint(-1, 2, (k, n), generator=gen).float()
    ref = a.double() @ w.double()
    guard = torch.full((m * n + 64,), 7.0, device=DEV)  # C is the front of this buffer: what lies behind it must stay
    c = guard[: m * n].view(m, n)
    from plexus_amd import _lib
    lib = _lib.load()
    ws, need = ops._split_ws(n, k, torch.device(DEV))
    ad, wd = a.to(DEV), w.to(DEV)
    _lib.check(lib.plx_gemm_nn_f32_split(m, n, k, ad.data_ptr(), k, wd.data_ptr(), n, c.data_ptr(), n, 0, ws.data_ptr(), need,
                                         torch.cuda.current_stream().cuda_stream), "plx_gemm_nn_f32_split")
    torch.cuda.synchronize()
    assert torch.equal(c.cpu().double(), ref) and bool((guard[m * n:] == 7.0).all())
    cb = ops.gemm_nt_bf16(bf(a).to(DEV), bf(w.t().contiguous()).to(DEV)).float().cpu()
    assert torch.equal(cb.double(), ref)  # |sum| <= 128: exact in bf16
    assert torch.equal(torch.relu(cb), ops.gemm_nt_bf16(bf(a).to(DEV), bf(w.t().contiguous()).to(DEV), relu=True).float().cpu())
