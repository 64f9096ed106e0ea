"""The torch.library form of the layer and the loss (plexus_amd/custom_ops.py): registration and shape propagation
on the CPU; on the GPU, bit-identity with the autograd-function path, the dispatcher's own operator checks, and
tracing without a graph break."""
import pytest
import torch

from plexus_amd import custom_ops as co


def test_operators_are_registered_and_propagate_shapes_without_a_gpu():
    from torch._subclasses.fake_tensor import FakeTensorMode

    for name in ("gcn_conv", "gcn_conv_bwd", "cross_entropy_fwd", "scale_by_scalar"):
        assert hasattr(torch.ops.plexus_amd, name)
    with FakeTensorMode():
        n, d_in, d_out, nnz = 50, 12, 5, 300
        i32 = dict(dtype=torch.int32)
        x = torch.empty(n * d_in)
        w = torch.empty(d_in * d_out)
        rp, ci, va = torch.empty(n + 1, **i32), torch.empty(nnz, **i32), torch.empty(nnz)
        out, agg = torch.ops.plexus_amd.gcn_conv(x, rp, ci, va, rp, ci, va, n, n, w, d_in, d_out, True)
        assert out.shape == (n, d_out) and agg.shape == (n, d_in)
        gx, gw = torch.ops.plexus_amd.gcn_conv_bwd(out, agg, out, w, rp, ci, va, n, n, d_in, d_out, True)
        assert gx.shape == (n, d_in) and gw.shape == w.shape
        loss, dl = torch.ops.plexus_amd.cross_entropy_fwd(out, torch.empty(n, dtype=torch.int64), n, d_out)
        assert loss.shape == () and dl.shape == out.shape


def _problem(dev):
    from plexus_amd import ops
    from plexus_amd.utils import synthetic as S

    n, dims = 1500, [40, 24, 7]
    g = S.build_graph(n, "chunglu", 20000, seed=2, device="cpu", gamma=2.1)
    a = ops.CsrMatrix(g.rowptr.to(dev), g.col.to(dev), g.val.to(dev), g.shape, 64)
    at = ops.CsrMatrix(g.rowptr_t.to(dev), g.col_t.to(dev), g.val_t.to(dev), g.shape, 64)
    ws = S.glorot_weights(dims, seed=1)
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(n * dims[0], generator=gen)
    y = torch.randint(0, dims[-1], (n,), generator=gen)
    return n, dims, a, at, ws, x, y


@pytest.mark.gpu
def test_custom_operators_match_the_autograd_functions_bit_for_bit():
    print("[case] torch.library operators against the autograd functions", flush=True)
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.train import Net

    dev = "cuda"
    n, dims, a, at, ws, x, y = _problem(dev)
    model = Net(2, dims[0], dims[1], dims[2], weights=ws, fuse_relu=True)
    x1 = x.to(dev).requires_grad_()
    (parallel_cross_entropy(model(x1, [(a, at)]), y.to(dev), 2, n, dims[-1]) * 2.0).backward()

    w = [t.clone().to(dev).requires_grad_() for t in ws]
    x2 = x.to(dev).requires_grad_()
    h = co.gcn_conv(x2, a, at, w[0], dims[0], dims[1], fuse_relu=True)
    out = co.gcn_conv(h, a, at, w[1], dims[1], dims[2])
    loss = co.cross_entropy(out, y.to(dev), n, dims[-1])
    (loss * 2.0).backward()
    assert torch.equal(x1.grad, x2.grad)
    for layer, wi in zip(model.layers, w):
        assert torch.equal(layer.weight.grad, wi.grad)


@pytest.mark.gpu
def test_dispatcher_checks_and_tracing_without_graph_breaks():
    print("[case] opcheck and torch.compile(fullgraph) of the custom operators", flush=True)
    dev = "cuda"
    n, dims, a, at, ws, x, y = _problem(dev)
    w0 = ws[0].to(dev).requires_grad_()
    xd = x.to(dev).requires_grad_()
    args = (xd, a.rowptr, a.col, a.val, at.rowptr, at.col, at.val, n, n, w0, dims[0], dims[1], True)
    co._parts(a), co._parts(at)
    checks = ("test_schema", "test_faketensor", "test_autograd_registration", "test_aot_dispatch_dynamic")
    torch.library.opcheck(torch.ops.plexus_amd.gcn_conv.default, args, test_utils=checks)
    logits = torch.randn(n, dims[-1], device=dev, requires_grad=True)
    torch.library.opcheck(torch.ops.plexus_amd.cross_entropy_fwd.default, (logits, y.to(dev), n, dims[-1]), test_utils=checks)

    w = [t.clone().to(dev).requires_grad_() for t in ws]
    yd = y.to(dev)

    arrays = (a.rowptr, a.col, a.val, at.rowptr, at.col, at.val)

    def step(x_in):  # the operators themselves: nothing but tensors and integers crosses the traced region
        h, _ = torch.ops.plexus_amd.gcn_conv(x_in, *arrays, n, n, w[0], dims[0], dims[1], True)
        out, _ = torch.ops.plexus_amd.gcn_conv(h, *arrays, n, n, w[1], dims[1], dims[2], False)
        return torch.ops.plexus_amd.cross_entropy_fwd(out, yd, n, dims[-1])[0]

    eager = step(xd)
    (g_eager,) = torch.autograd.grad(eager, xd)
    compiled = torch.compile(step, backend="aot_eager", fullgraph=True)
    traced = compiled(xd)
    (g_traced,) = torch.autograd.grad(traced, xd)
    assert torch.equal(eager, traced) and torch.equal(g_eager, g_traced)


@pytest.mark.gpu
def test_plan_cache_never_serves_another_matrix_and_sees_in_place_edits():
    """The prepared form of a matrix is cached under the addresses of the caller's arrays.  int64 indices (what torch CSR
    tensors carry) and non-fp32 values are converted to copies, so the caller's arrays can be dropped while the entry
    lives: a later matrix of the same shape and entry count must still get its own product, an in-place edit of the
    values must be seen, and the cache stays bounded."""
    print("[case] plan cache of the custom operators: freed arrays, same-size successor, in-place edit, bound", flush=True)
    dev = "cuda"
    co.clear_plan_cache()
    n, d_in, d_out, nnz = 400, 16, 8, 3000
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, d_in, generator=gen)
    w = torch.randn(d_in, d_out, generator=gen)

    def random_csr(seed):
        g = torch.Generator().manual_seed(seed)
        flat = torch.randperm(n * n, generator=g)[:nnz].sort().values  # nnz distinct positions: every matrix has exactly nnz entries
        rows, cols = flat // n, flat % n
        rowptr = torch.zeros(n + 1, dtype=torch.int64)
        rowptr[1:] = torch.cumsum(torch.bincount(rows, minlength=n), 0)
        return rowptr, cols, torch.rand(nnz, generator=g, dtype=torch.float64) + 0.5

    def run(rowptr, col, val):
        out, _ = torch.ops.plexus_amd.gcn_conv(x.to(dev).reshape(-1), rowptr, col, val, rowptr, col, val, n, n, w.to(dev).reshape(-1),
                                               d_in, d_out, False)
        return out.cpu()

    def expect(rowptr, col, val):
        a = torch.sparse_csr_tensor(rowptr, col, val.float(), size=(n, n))
        return torch.mm(torch.sparse.mm(a, x), w)

    for seed in range(3):  # each round drops the previous arrays before allocating arrays of the same sizes
        rowptr, col, val = random_csr(seed)
        rd, cd, vd = rowptr.to(dev), col.to(dev), val.to(dev)
        assert torch.allclose(run(rd, cd, vd), expect(rowptr, col, val), rtol=1e-5, atol=1e-5), "matrix %d" % seed
        if seed == 2:  # values edited in place (the prepared matrix holds an fp32 copy of these fp64 values)
            vd.mul_(2.0)
            assert torch.allclose(run(rd, cd, vd), 2.0 * expect(rowptr, col, val), rtol=1e-5, atol=1e-5)
            cd.copy_(torch.flip(cd, [0]) * 0 + cd)  # an in-place write that leaves the structure as it is: still a valid plan
            assert torch.allclose(run(rd, cd, vd), 2.0 * expect(rowptr, col, val), rtol=1e-5, atol=1e-5)
        del rd, cd, vd
    keep = []
    for seed in range(co.MAX_PLANS + 3):
        rowptr, col, val = random_csr(100 + seed)
        keep.append((rowptr.to(dev), col.to(dev), val.to(dev)))
        run(*keep[-1])
    assert len(co._PLANS) == co.MAX_PLANS
    rowptr, col, val = random_csr(100)  # evicted meanwhile: prepared again, same result
    assert torch.allclose(run(*keep[0]), expect(rowptr, col, val), rtol=1e-5, atol=1e-5)
    co.clear_plan_cache()
