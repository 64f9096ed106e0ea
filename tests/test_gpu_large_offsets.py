"""Dense matrices of more than 2^31 elements: every element offset inside the kernels has to be 64-bit.

The matrices have 2^24 + 1000 rows of 128 columns (8.6 GB in fp32).  Row blocks at the start, around the 2^31-element
mark and at the end are compared with fp64 arithmetic by torch on the same device; reductions over all rows are
compared in full.
"""
import pytest
import torch

from conftest import BF16_TOL, FP32_TOL, rel_err
from plexus_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
M = 2 ** 24 + 1000
D = 128
BLOCK = 4096
# the element with linear index 2^31 sits in row 2^24
STARTS = [0, 2 ** 24 - BLOCK + 500, M - BLOCK]


def say(msg):
    print("[case] " + msg, flush=True)


def blocks(*tensors):
    for r0 in STARTS:
        yield tuple(t[r0:r0 + BLOCK] for t in tensors)


@pytest.fixture(scope="module")
def operands():
    gen = torch.Generator(device=DEV).manual_seed(0)
    a = torch.randn(M, D, device=DEV, generator=gen)
    g = torch.randn(M, D, device=DEV, generator=gen)
    w = torch.randn(D, D, device=DEV, generator=gen) * 0.1
    assert a.numel() > 2 ** 31
    yield a, g, w
    del a, g, w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("path", ["split", "mfma32"])
def test_fp32_products(operands, path):
    say("fp32 products on 2^31+ elements, %s" % path)
    a, g, w = operands
    keep = ops.SPLIT_GEMM
    ops.SPLIT_GEMM = path == "split"
    try:
        out = ops.gemm_nn(a, w, relu=True)
        for ab, ob in blocks(a, out):
            assert rel_err(ob, torch.relu(ab.double() @ w.double())) <= FP32_TOL
        dagg = ops.gemm_nt(g, w, mask=out)
        for gb, ob, db in blocks(g, out, dagg):
            assert rel_err(db, (gb.double() * (ob > 0)) @ w.double().t()) <= FP32_TOL
        del dagg
        if path == "split":  # the reduction over all rows has one implementation
            dw = ops.gemm_tn(a, g, mask=out)
            ref = torch.zeros(D, D, dtype=torch.float64, device=DEV)
            step = 2 ** 20
            for r0 in range(0, M, step):
                ref += a[r0:r0 + step].double().t() @ (g[r0:r0 + step].double() * (out[r0:r0 + step] > 0))
            assert rel_err(dw, ref) <= FP32_TOL
    finally:
        ops.SPLIT_GEMM = keep


def test_relu_and_cross_entropy(operands):
    say("relu, relu backward and cross-entropy on 2^31+ elements")
    a, g, _ = operands
    y = ops.relu(a)
    dx = ops.relu_bwd(g, y)
    for ab, gb, yb, db in blocks(a, g, y, dx):
        assert torch.equal(yb, torch.relu(ab)) and torch.equal(db, gb * (ab > 0))
    del y, dx
    labels = torch.randint(0, D, (M,), device=DEV, generator=torch.Generator(device=DEV).manual_seed(1))
    labels[2 ** 24 + 5] = -1
    loss, dl = ops.softmax_xent(a, labels, M, D)
    total = torch.zeros((), dtype=torch.float64, device=DEV)
    step = 2 ** 20
    for r0 in range(0, M, step):
        lb = labels[r0:r0 + step]
        lp = torch.log_softmax(a[r0:r0 + step].double(), dim=1)
        picked = lp.gather(1, lb.clamp(min=0)[:, None])[:, 0]
        total -= torch.where(lb >= 0, picked, torch.zeros_like(picked)).sum()
    assert abs(loss.item() - (total / M).item()) <= FP32_TOL * abs((total / M).item())
    for ab, lb, db in blocks(a, labels[:, None], dl):
        sm = torch.softmax(ab.double(), dim=1)
        onehot = torch.zeros_like(sm).scatter_(1, lb.clamp(min=0), 1.0)
        ref = torch.where(lb >= 0, (sm - onehot) / M, torch.zeros_like(sm))
        assert rel_err(db, ref) <= FP32_TOL


def test_cross_entropy_odd_width_contiguous_rows():
    say("cross-entropy, 47 classes, 46 M rows (2^31+ elements)")
    m, c = 46_000_000, 47
    gen = torch.Generator(device=DEV).manual_seed(2)
    x = torch.randn(m, c, device=DEV, generator=gen)
    assert x.numel() > 2 ** 31
    labels = torch.randint(0, c, (m,), device=DEV, generator=gen)
    loss, dl = ops.softmax_xent(x, labels, m, c)
    total = torch.zeros((), dtype=torch.float64, device=DEV)
    step = 2 ** 21
    for r0 in range(0, m, step):
        lp = torch.log_softmax(x[r0:r0 + step].double(), dim=1)
        total -= lp.gather(1, labels[r0:r0 + step, None]).sum()
    assert abs(loss.item() - (total / m).item()) <= FP32_TOL * abs((total / m).item())
    for r0 in (0, 2 ** 31 // c - BLOCK // 2, m - BLOCK):
        sm = torch.softmax(x[r0:r0 + BLOCK].double(), dim=1)
        ref = (sm - torch.zeros_like(sm).scatter_(1, labels[r0:r0 + BLOCK, None], 1.0)) / m
        assert rel_err(dl[r0:r0 + BLOCK], ref) <= FP32_TOL
    del x, dl
    torch.cuda.empty_cache()


def test_adamw(operands):
    say("AdamW over 2^31+ elements")
    from plexus_amd.optim import AdamW

    a, g, _ = operands
    p = a.clone().reshape(-1).requires_grad_()
    p.grad = g.reshape(-1)
    opt = AdamW([p], lr=3e-3, weight_decay=0.01)
    opt.step()
    n = p.numel()
    for e0 in (0, 2 ** 31 - 2 ** 19, n - 2 ** 20):
        sl = slice(e0, e0 + 2 ** 20)
        p0, gr = a.reshape(-1)[sl].double(), g.reshape(-1)[sl].double()
        m1, v1 = 0.1 * gr, 0.001 * gr * gr
        ref = p0 * (1 - 3e-3 * 0.01) - 3e-3 / (1 - 0.9) * m1 / (v1.sqrt() / (1 - 0.999) ** 0.5 + 1e-8)
        assert rel_err(p.detach()[sl], ref) <= FP32_TOL
        assert rel_err(opt.state[p]["exp_avg"][sl], m1) <= FP32_TOL and rel_err(opt.state[p]["exp_avg_sq"][sl], v1) <= FP32_TOL
    del p, opt
    torch.cuda.empty_cache()


def test_bf16_products_and_cast(operands):
    say("bf16 products on 2^31+ elements")
    a, g, w = operands
    ab, gb = ops.cast_bf16(a), ops.cast_bf16(g)
    for x32, x16 in blocks(a, ab):
        assert torch.equal(x16, x32.to(torch.bfloat16))
    wt = ops.cast_bf16(w, transpose=True)  # [out x in]
    out = ops.gemm_nt_bf16(ab, wt, relu=True)
    for x16, ob in blocks(ab, out):
        assert rel_err(ob.float(), torch.relu(x16.double() @ wt.double().t())) <= BF16_TOL
    wb = ops.cast_bf16(w)  # [in x out]
    dagg = ops.gemm_nt_bf16(gb, wb, mask=out)
    for g16, ob, db in blocks(gb, out, dagg):
        assert rel_err(db.float(), (g16.double() * (ob > 0)) @ wb.double().t()) <= BF16_TOL
    del dagg
    dw = ops.gemm_tn_bf16(ab, gb, mask=out)
    ref = torch.zeros(D, D, dtype=torch.float64, device=DEV)
    step = 2 ** 20
    for r0 in range(0, M, step):
        ref += ab[r0:r0 + step].double().t() @ (gb[r0:r0 + step].double() * (out[r0:r0 + step] > 0))
    assert rel_err(dw, ref) <= FP32_TOL  # fp32 accumulation of exact bf16 products
    labels = torch.randint(0, D, (M,), device=DEV, generator=torch.Generator(device=DEV).manual_seed(3))
    loss, dl = ops.softmax_xent(out, labels, M, D)
    for ob, lb, db in blocks(out, labels[:, None], dl):
        sm = torch.softmax(ob.double(), dim=1)
        ref_b = (sm - torch.zeros_like(sm).scatter_(1, lb, 1.0)) / M
        assert rel_err(db.float(), ref_b) <= BF16_TOL
    assert torch.isfinite(loss).all()


def test_spmm_output_beyond_2_31_elements():
    say("SpMM whose output holds 2^31+ elements")
    k, per_row = 2 ** 20, 4
    gen = torch.Generator(device=DEV).manual_seed(4)
    col = torch.randint(0, k, (M, per_row), dtype=torch.int32, device=DEV, generator=gen).reshape(-1)
    val = torch.rand(M * per_row, device=DEV, generator=gen)
    rowptr = (torch.arange(M + 1, dtype=torch.int64, device=DEV) * per_row).to(torch.int32)
    a = ops.CsrMatrix(rowptr, col, val, (M, k))
    h = torch.randn(k, D, device=DEV, generator=gen)
    y = ops.spmm(a, h)
    assert y.numel() > 2 ** 31
    for r0 in STARTS:
        c = col[r0 * per_row:(r0 + BLOCK) * per_row].long()
        ref = (h[c].double().view(BLOCK, per_row, D) * val[r0 * per_row:(r0 + BLOCK) * per_row].double().view(BLOCK, per_row, 1)).sum(1)
        assert rel_err(y[r0:r0 + BLOCK], ref) <= FP32_TOL
