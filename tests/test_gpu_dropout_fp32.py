"""Fused dropout with fp32 storage: the mask of the fp32 forward product is the oracle's bit for bit, its scale enters
the backward products once, and a three-layer network with it follows the oracle network.

fp32 bar: max|x - ref| / max|ref| <= 1e-5 per output tensor.
"""
import ctypes

import pytest
import torch

from conftest import FP32_TOL, rel_err
from oracle import oracle_c
from oracle import plexus_oracle as po
from plexus_amd import _lib, ops
from plexus_amd.utils import synthetic as S

pytestmark = pytest.mark.gpu
DEV = "cuda"


def say(msg):
    print("[case] " + msg, flush=True)


def _pack_bits(x):
    m, n = x.shape
    words = (n + 31) // 32
    pos = torch.zeros(m, words * 32, dtype=torch.int64)
    pos[:, :n] = (x > 0).to(torch.int64)
    w = (pos.reshape(m, words, 32) << torch.arange(32, dtype=torch.int64)).sum(-1)
    return torch.where(w >= 2**31, w - 2**32, w).to(torch.int32)


# resident kernel with the mask applied to the accumulators (N % 8 == 0, weights <= 128 x 128): one, two and four column
# tiles, a last panel of fewer than 32 rows; resident kernel + pass over C (N % 8 != 0); weights beyond 128 x 128 (pass
# over C); operands the split products do not take (fp32 MFMA + plx_dropout_f32)
@pytest.mark.parametrize("m,n,k", [(3000, 128, 100), (1001, 128, 128), (515, 64, 128), (77, 24, 16), (2050, 96, 64), (777, 47, 128),
                                   (300, 100, 60), (500, 200, 150), (129, 131, 7)])
@pytest.mark.parametrize("p", [0.5, 0.25])
def test_fp32_dropout_mask_is_the_oracles(m, n, k, p):
    say("fp32 fused dropout %dx%dx%d p=%g" % (m, n, k, p))
    gen = torch.Generator().manual_seed(m + n)
    a = torch.rand(m, k, generator=gen) + 0.1  # positive products: every kept element is > 0
    w = torch.rand(k, n, generator=gen) + 0.1
    seed, offset = 1234567890123, 77
    c, bits = ops.gemm_nn(a.to(DEV), w.to(DEV), relu=True, want_bits=True, dropout_p=p, seed=seed, offset=offset)
    c = c.cpu()
    keep = torch.from_numpy(po.dropout_keep_mask(m * n, seed, offset, p).reshape(m, n))
    assert torch.equal(c > 0, keep)  # bit-exact mask
    assert abs(keep.float().mean().item() - (1 - p)) < 0.03
    ref = oracle_c.gemm(a.numpy(), w.numpy()) * keep.numpy() / (1 - p)
    assert rel_err(c, ref) <= FP32_TOL
    assert torch.equal(bits.cpu(), _pack_bits(c))  # the bits are those of the dropped-out result
    # without the bits, and with another offset
    c1 = ops.gemm_nn(a.to(DEV), w.to(DEV), relu=True, dropout_p=p, seed=seed, offset=offset).cpu()
    assert torch.equal(c1, c)
    c2 = ops.gemm_nn(a.to(DEV), w.to(DEV), relu=True, dropout_p=p, seed=seed, offset=offset + 1).cpu()
    assert not torch.equal(c2 > 0, keep)
    # the kept elements are the product without dropout times 1 / (1 - p), up to the rounding of that product
    plain = ops.gemm_nn(a.to(DEV), w.to(DEV), relu=True).cpu()
    assert rel_err(c, plain * keep / (1 - p)) <= 2e-7
    # the stand-alone kernel applies the same mask
    x = plain.clone().to(DEV)
    ops.dropout_(x, p, seed, offset)
    assert torch.equal(x.cpu() > 0, keep) and rel_err(x.cpu(), c) <= 2e-7


def test_fp32_dropout_of_a_product_the_guarded_launch_redoes():
    say("fp32 fused dropout when an operand holds Inf (the fp32 kernel redoes the product, the mask is applied to that)")
    gen = torch.Generator().manual_seed(9)
    m, n, k, p = 700, 128, 128, 0.5
    a = torch.rand(m, k, generator=gen) + 0.1
    a[5, 3] = float("inf")
    w = torch.rand(k, n, generator=gen) + 0.1
    c, bits = ops.gemm_nn(a.to(DEV), w.to(DEV), relu=True, want_bits=True, dropout_p=p, seed=3, offset=4)
    c = c.cpu()
    keep = torch.from_numpy(po.dropout_keep_mask(m * n, 3, 4, p).reshape(m, n))
    assert torch.equal(c > 0, keep)
    assert torch.isinf(c[5][keep[5]]).all() and (c[5][~keep[5]] == 0).all()
    assert torch.equal(bits.cpu(), _pack_bits(c))


def test_fp32_entry_points_without_dropout_arguments_refuse_the_flag():
    say("PLX_GEMM_DROPOUT on fp32 entry points that carry no p / seed / offset")
    lib = _lib.load()
    a = torch.randn(64, 32, device=DEV)
    w = torch.randn(32, 16, device=DEV)
    c = torch.empty(64, 16, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.plx_gemm_nn_f32(64, 16, 32, a.data_ptr(), 32, w.data_ptr(), 16, c.data_ptr(), 16, _lib.PLX_GEMM_RELU | _lib.PLX_GEMM_DROPOUT, st)
    assert rc == _lib.PLX_ERR_UNSUPPORTED and b"DROPOUT" in lib.plx_last_error()
    need = int(lib.plx_gemm_f32_split_workspace_bytes(16, 32))
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    rc = lib.plx_gemm_nn_f32_split(64, 16, 32, a.data_ptr(), 32, w.data_ptr(), 16, c.data_ptr(), 16, _lib.PLX_GEMM_DROPOUT, ws.data_ptr(), need, st)
    assert rc == _lib.PLX_ERR_UNSUPPORTED
    bits = torch.empty(64, 4, dtype=torch.int32, device=DEV)
    rc = lib.plx_gemm_nn_f32_split_bits(64, 16, 32, a.data_ptr(), 32, w.data_ptr(), 16, c.data_ptr(), 16, _lib.PLX_GEMM_DROPOUT,
                                        bits.data_ptr(), 4, ws.data_ptr(), need, st)
    assert rc == _lib.PLX_ERR_UNSUPPORTED
    # p outside [0, 1) is an argument error of the entry point that does take it
    rc = lib.plx_gemm_nn_f32_split_dropout(64, 16, 32, a.data_ptr(), 32, w.data_ptr(), 16, c.data_ptr(), 16, _lib.PLX_GEMM_DROPOUT,
                                           ctypes.c_float(1.0), 1, 2, None, 0, ws.data_ptr(), need, st)
    assert rc == _lib.PLX_ERR_INVALID


@pytest.mark.parametrize("m,n,k", [(3000, 128, 100), (777, 47, 128), (500, 200, 150)])
def test_backward_products_scaled_by_the_dropout_factor(m, n, k):
    say("GRAD_AGG and GRAD_W with alpha, %dx%dx%d" % (m, n, k))
    gen = torch.Generator().manual_seed(m + k)
    gout = torch.randn(m, n, generator=gen)
    w = torch.randn(k, n, generator=gen) * 0.1
    act = torch.relu(torch.randn(m, n, generator=gen))
    agg = torch.randn(m, k, generator=gen)
    bits = ops.sign_bits(act.to(DEV))
    for alpha in (2.0, 1.0 / 0.75):
        got = ops.gemm_nt(gout.to(DEV), w.to(DEV), mask=act.to(DEV), mask_bits=bits, alpha=alpha).cpu()
        ref = alpha * oracle_c.gemm((gout * (act > 0)).numpy(), w.numpy(), tb=True)
        assert rel_err(got, ref) <= FP32_TOL
        gw = ops.gemm_tn(agg.to(DEV), gout.to(DEV), mask=act.to(DEV), alpha=alpha).cpu()
        assert rel_err(gw, alpha * oracle_c.gemm(agg.numpy(), (gout * (act > 0)).numpy(), ta=True)) <= FP32_TOL
    # a power of two scales the unscaled product exactly; alpha = 1 is that product
    one = ops.gemm_nt(gout.to(DEV), w.to(DEV), mask=act.to(DEV), mask_bits=bits)
    assert torch.equal(ops.gemm_nt(gout.to(DEV), w.to(DEV), mask=act.to(DEV), mask_bits=bits, alpha=2.0), 2.0 * one)


def test_fp32_three_layer_network_with_dropout_follows_the_oracle():
    """100-128-128-47 at 1/100 of the 2.45 M-node graph, fp32 storage, dropout 0.5 after each ReLU: forward, loss and
    backward against the fp32 oracle network with the same masks (regenerated on the host from seed and offsets)."""
    say("fp32 network with dropout 0.5 at 1/100 scale")
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.train import Net

    g = S.config3_graph("cpu", seed=1, scale=0.01)
    n = g.shape[0]
    dims = [100, 128, 128, 47]
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, dims[0], generator=gen)
    y = torch.randint(0, 47, (n,), generator=gen)
    ws = S.glorot_weights(dims, seed=2)
    seed = 42
    model = Net(3, dims[0], dims[1], dims[-1], weights=ws, fuse_relu=True, dropout=0.5, dropout_seed=seed)
    model.train()
    offsets = [layer.next_dropout_offset() for layer in model.layers]
    shards = [(ops.CsrMatrix(g.rowptr.to(DEV), g.col.to(DEV), g.val.to(DEV), g.shape),
               ops.CsrMatrix(g.rowptr_t.to(DEV), g.col_t.to(DEV), g.val_t.to(DEV), (g.shape[1], g.shape[0])))]
    xd = x.reshape(-1).to(DEV).requires_grad_()
    logits = model(xd, shards)
    loss = parallel_cross_entropy(logits, y.to(DEV), 3, n, 47)
    loss.backward()

    adj = [(g.torch_csr(), g.torch_csr(True))]
    for dtype in (torch.float32, torch.float64):
        net = po.OracleNet([w.to(dtype) for w in ws], dims, dropout_p=0.5, seed=seed)
        ref_logits = net.forward(x.reshape(-1).to(dtype), [(a.to(dtype), b.to(dtype)) for a, b in adj], offsets)
        ref_loss, sm, oh = po.cross_entropy_forward(ref_logits, y, n, 47)
        gl = po.cross_entropy_backward(sm, oh.to(dtype), n)
        gx_ref, gws_ref = net.backward(gl)
        assert rel_err(logits, ref_logits) <= FP32_TOL
        assert abs(loss.item() - ref_loss.item()) <= FP32_TOL * abs(ref_loss.item())
        assert rel_err(xd.grad, gx_ref) <= FP32_TOL
        for layer, gw in zip(model.layers, gws_ref):
            assert rel_err(layer.weight.grad, gw) <= FP32_TOL
    # the masks dropped about half of the live units, and a second forward draws other masks
    hidden_keep = torch.from_numpy(po.dropout_keep_mask(n * 128, seed, offsets[0], 0.5))
    assert 0.45 < hidden_keep.float().mean().item() < 0.55
    logits2 = model(xd.detach(), shards)
    assert not torch.equal(logits2, logits)
    model.eval()
    assert torch.equal(model(xd.detach(), shards), model(xd.detach(), shards))
