"""Pins the CPU oracle (oracle/) without the reference: the reference has no tests or golden vectors
for this path, so each oracle function is checked against something the mathematics fixes --
dense products, scipy, brute-force loops, library closed forms, autograd, published known answers."""
import math

import numpy as np
import pytest
import scipy.sparse as sp
import torch
import torch.nn.functional as F

from oracle import oracle_c
from oracle import plexus_oracle as po
from plexus_amd.utils import synthetic as S


def small_graph(n=97, pairs=400, seed=3, with_empty_rows=True):
    g = torch.Generator().manual_seed(seed)
    src = torch.randint(0, n, (pairs,), generator=g)
    dst = torch.randint(0, n, (pairs,), generator=g)
    if with_empty_rows:
        keep = (src % 7 != 0)
        src, dst = src[keep], dst[keep]
    w = torch.rand(src.numel(), generator=g) + 0.1
    a = torch.sparse_coo_tensor(torch.stack([src, dst]), w, (n, n)).coalesce()
    return a.to_sparse_csr()


def brute_spmm(crow, col, val, h):
    m = len(crow) - 1
    y = np.zeros((m, h.shape[1]), dtype=np.float64)
    for r in range(m):
        for j in range(crow[r], crow[r + 1]):
            for d in range(h.shape[1]):
                y[r, d] += float(val[j]) * float(h[col[j], d])
    return y


def test_spmm_oracle_vs_dense_scipy_bruteforce():
    a = small_graph()
    h = torch.randn(97, 13, generator=torch.Generator().manual_seed(1))
    y = po.spmm(a, h)
    dense = a.to_dense().double() @ h.double()
    assert torch.allclose(y.double(), dense, rtol=0, atol=1e-5)
    crow, col, val = a.crow_indices().numpy(), a.col_indices().numpy(), a.values().numpy()
    ys = sp.csr_matrix((val.astype(np.float64), col, crow), shape=(97, 97)) @ h.double().numpy()
    assert np.allclose(dense.numpy(), ys, atol=1e-12)
    yb = brute_spmm(crow, col, val, h.numpy())
    assert np.allclose(dense.numpy(), yb, atol=1e-12)
    # the C restatement: fp64 accumulation, fp32 accumulation, and all-fp64
    assert np.allclose(oracle_c.csr_spmm(crow, col, val, h.numpy(), acc64=True), dense.numpy(), atol=2e-6)
    assert np.allclose(oracle_c.csr_spmm(crow, col, val, h.numpy(), acc64=False), dense.numpy(), atol=1e-5)
    assert np.allclose(oracle_c.csr_spmm(crow, col, val.astype(np.float64), h.double().numpy()), dense.numpy(), atol=1e-12)


def test_spmm_oracle_invariants():
    a = small_graph(n=120, pairs=900, seed=5)
    n = 120
    g = torch.Generator().manual_seed(2)
    # A.1 = row sums ; empty row -> zero row
    ones = torch.ones(n, 3)
    y = po.spmm(a, ones)
    crow = a.crow_indices()
    rowsum = torch.zeros(n).index_add_(0, torch.repeat_interleave(torch.arange(n), crow[1:] - crow[:-1]), a.values())
    assert torch.allclose(y[:, 0], rowsum, atol=1e-5)
    empty = (crow[1:] - crow[:-1]) == 0
    assert empty.any() and (y[empty] == 0).all()
    # adjoint identity <A.H, G> = <H, A^T.G> with the separately materialised transpose
    a_t = a.transpose(0, 1).to_sparse_csr()
    h = torch.randn(n, 6, generator=g, dtype=torch.float64)
    gg = torch.randn(n, 6, generator=g, dtype=torch.float64)
    a64, a_t64 = a.double(), a_t.double()
    lhs = (po.spmm(a64, h) * gg).sum()
    rhs = (h * po.spmm(a_t64, gg)).sum()
    assert abs(lhs - rhs) < 1e-9 * abs(lhs)
    # permutation equivariance (P A Q^T)(Q H) = P (A H)
    p, q = torch.randperm(n, generator=g), torch.randperm(n, generator=g)
    dense = a64.to_dense()
    paq = torch.zeros_like(dense)
    paq[p[:, None], q[None, :]] = dense
    qh = torch.zeros_like(h)
    qh[q] = h
    ref = torch.zeros_like(h)
    ref[p] = po.spmm(a64, h)
    assert torch.allclose(po.spmm(paq.to_sparse_csr(), qh), ref, atol=1e-12)


def test_chunked_spmm_equals_unchunked():
    a = small_graph(n=103, pairs=700, seed=8)
    h = torch.randn(103, 5, generator=torch.Generator().manual_seed(4))
    assert po.chunk_bounds(2449029) == [(0, 816343), (816343, 1632686), (1632686, 2449029)]
    assert po.chunk_bounds(10, 4) == [(0, 3), (3, 6), (6, 10)]
    assert torch.equal(po.chunked_spmm(a, h, max_rows_per_chunk=10), po.spmm(a, h))


def test_gemm_c_oracle_vs_numpy():
    rng = np.random.default_rng(0)
    a = rng.standard_normal((37, 21)).astype(np.float32)
    b = rng.standard_normal((21, 11)).astype(np.float32)
    assert np.allclose(oracle_c.gemm(a, b), a.astype(np.float64) @ b.astype(np.float64), atol=1e-5)
    g = rng.standard_normal((37, 11)).astype(np.float32)
    assert np.allclose(oracle_c.gemm(a, g, ta=True), a.astype(np.float64).T @ g, atol=1e-5)
    w = rng.standard_normal((21, 11)).astype(np.float32)
    assert np.allclose(oracle_c.gemm(g, w, tb=True), g.astype(np.float64) @ w.astype(np.float64).T, atol=1e-5)


def test_layer_backward_formulas_vs_autograd():
    """The hand formulas of gcn_conv.py:236-266 equal autograd over the plain-operator forward."""
    n, din, dout = 60, 9, 5
    a = small_graph(n=n, pairs=300, seed=11).double()
    a_t = a.transpose(0, 1).to_sparse_csr()
    g = torch.Generator().manual_seed(6)
    x = torch.randn(n * din, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(din * dout, generator=g, dtype=torch.float64, requires_grad=True)
    out, agg = po.gcn_conv_forward(x, a, w, (n, din), (din, dout))
    go = torch.randn(n, dout, generator=g, dtype=torch.float64)
    gx_ref, gw_ref = torch.autograd.grad(out, [x, w], go)
    gx, gw = po.gcn_conv_backward(go, agg.detach(), w.detach(), a_t, (din, dout), flatten_grad_x=True)
    assert torch.allclose(gx, gx_ref, atol=1e-12) and gx.shape == x.shape
    assert torch.allclose(gw, gw_ref, atol=1e-12) and gw.shape == w.shape
    # and the forward equals the dense product
    ref = (a.to_dense() @ x.detach().reshape(n, din)) @ w.detach().reshape(din, dout)
    assert torch.allclose(out.detach(), ref, atol=1e-12)


def test_cross_entropy_equals_library_mean_loss():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(50, 11, generator=g, dtype=torch.float64)
    y = torch.randint(0, 11, (50,), generator=g)
    loss, softmax, onehot = po.cross_entropy_forward(logits, y, 50, 11)
    lg = logits.clone().requires_grad_()
    ref = F.cross_entropy(lg, y)
    assert abs(loss - ref) < 1e-12
    (gref,) = torch.autograd.grad(ref, lg)
    grad = po.cross_entropy_backward(softmax, onehot.double(), 50)
    assert torch.allclose(grad, gref, atol=1e-14)
    assert torch.allclose(grad.sum(1), torch.zeros(50, dtype=torch.float64), atol=1e-15)
    # inputs untouched
    assert torch.equal(logits, lg.detach())
    # C restatement agrees (fp32 logits)
    l32 = logits.float()
    closs, cgrad = oracle_c.softmax_xent(l32.numpy(), y.numpy(), 50, 11)
    ref32 = F.cross_entropy(l32.double(), y)
    assert abs(closs - ref32) < 1e-9
    assert np.allclose(cgrad, po.cross_entropy_backward(*[t.double() for t in po.cross_entropy_forward(l32.double(), y, 50, 11)[1:]], 50).numpy(), atol=1e-8)


def test_cross_entropy_special_cases():
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(8, 6, generator=g, dtype=torch.float64)
    y = torch.tensor([0, 1, -1, 3, 5, 2, 0, 4])
    num_nodes, num_classes = 6, 5  # rows 6,7 are padded; class 5 is padded
    loss, softmax, onehot = po.cross_entropy_forward(logits, y, num_nodes, num_classes)
    grad = po.cross_entropy_backward(softmax, onehot.double(), num_nodes)
    # label < 0: zero loss, zero gradient row
    assert (softmax[2] == 0).all() and (grad[2] == 0).all()
    # padded class has probability 0 everywhere
    assert (softmax[:, 5] == 0).all()
    # rows past num_nodes: softmax zero; label 0 / 4 is valid so each adds -log(1e-9)
    assert (softmax[6:] == 0).all()
    # row 4 is labelled with the padded class: probability 0 -> -log(1e-9) as well
    valid = [0, 1, 3, 5]
    sm = torch.softmax(logits[:, :5], dim=1)
    expect = sum(-math.log(sm[i, y[i]]) for i in valid) + 3 * (-math.log(1e-9))
    assert abs(loss * num_nodes - expect) < 1e-10
    assert abs(-math.log(1e-9) - 20.7233) < 1e-4
    # valid rows: gradient rows sum to zero
    assert torch.allclose(grad[valid].sum(1), torch.zeros(4, dtype=torch.float64), atol=1e-15)
    closs, cgrad = oracle_c.softmax_xent(logits.float().numpy(), y.numpy(), num_nodes, num_classes)
    l32, s32, o32 = po.cross_entropy_forward(logits.float().double(), y, num_nodes, num_classes)
    assert abs(closs - l32) < 1e-9
    assert np.allclose(cgrad, po.cross_entropy_backward(s32, o32.double(), num_nodes).numpy(), atol=1e-8)


def test_gcn_norm_closed_forms():
    # ring of n nodes, each linked to its k nearest on both sides: (2k)-regular -> every entry 1 / (2k + 1)
    n, k = 30, 2
    src = torch.arange(n).repeat_interleave(2 * k)
    off = torch.tensor([-2, -1, 1, 2]).repeat(n)
    dst = (src + off) % n
    ei, w = po.gcn_norm(torch.stack([src, dst]), n)
    assert ei.shape[1] == n * (2 * k + 1)
    assert torch.allclose(w, torch.full_like(w, 1.0 / (2 * k + 1)))
    # general symmetric graph: dense formula D^-1/2 (A + I) D^-1/2, symmetric result
    g = S.build_graph(40, "uniform", 0, seed=1, permute=False, exact_pairs=90)
    dense = g.torch_csr().to_dense().double()
    adj = (dense != 0).double()
    d = adj.sum(1)
    ref = adj / torch.sqrt(d[:, None] * d[None, :])
    assert torch.allclose(dense, ref, atol=1e-7)
    assert torch.equal(dense, dense.t())
    # CSR-values variant and the C restatement reproduce it from unit values
    ones = torch.ones_like(g.val)
    v = po.gcn_norm_csr_values(g.rowptr, g.col, ones)
    assert torch.allclose(v, g.val, atol=1e-7)
    vc = oracle_c.gcn_norm_csr(g.rowptr.numpy(), g.col.numpy(), ones.numpy())
    assert np.allclose(vc, g.val.numpy(), atol=1e-7)
    # PyG-style edge-list variant agrees on the same graph without its loops
    crow = g.rowptr
    rows = torch.repeat_interleave(torch.arange(40), crow[1:] - crow[:-1])
    nl = rows != g.col
    ei2, w2 = po.gcn_norm(torch.stack([rows[nl], g.col[nl]]), 40)
    d2 = torch.zeros(40, 40, dtype=torch.float64)
    d2[ei2[0], ei2[1]] = w2.double()
    assert torch.allclose(d2, ref, atol=1e-7)


def test_weight_init_bound():
    w = po.kaiming_uniform_weight(100, 16, torch.Generator().manual_seed(0))
    assert w.shape == (1600,)
    assert w.abs().max() <= 1 / math.sqrt(16) and w.abs().max() > 0.24
    assert abs(w.mean()) < 0.02
    # same bound as torch's initialiser on an (in, out) tensor: fan_in = size(1)
    t = torch.empty(100, 16)
    torch.manual_seed(0)
    torch.nn.init.kaiming_uniform_(t, a=math.sqrt(5))
    assert t.abs().max() <= 1 / math.sqrt(16) and t.abs().max() > 0.24


def test_philox_known_answers():
    """Published Random123 known-answer vectors for philox4x32-10."""
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
        ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
        ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
         (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
    ]
    for ctr, key, out in kat:
        r = po.philox4x32_10(np.array([ctr], dtype=np.uint32), key)
        assert tuple(int(v) for v in r[0]) == out
    m = po.dropout_keep_mask(100000, seed=0, offset=3, p=0.5)
    assert abs(m.mean() - 0.5) < 0.01
    assert abs(po.dropout_keep_mask(100000, seed=0, offset=3, p=0.25).mean() - 0.75) < 0.01
    assert po.dropout_keep_mask(1000, 1, 0, 0.0).all()


def test_adamw_step_matches_torch():
    g = torch.Generator().manual_seed(0)
    p0 = [torch.randn(7, generator=g, dtype=torch.float64), torch.randn(3, 4, generator=g, dtype=torch.float64)]
    params = [p.clone().requires_grad_() for p in p0]
    opt = torch.optim.AdamW(params, lr=3e-3, weight_decay=0.0)
    mine = [p.clone() for p in p0]
    state = {}
    for _ in range(4):
        grads = [torch.randn(p.shape, generator=g, dtype=torch.float64) for p in p0]
        for p, gr in zip(params, grads):
            p.grad = gr.clone()
        opt.step()
        po.adamw_step(mine, grads, state, lr=3e-3)
    for a, b in zip(mine, params):
        assert torch.allclose(a, b.detach(), atol=1e-12)


def test_epoch_loop_matches_autograd_training():
    """OracleNet + hand backward + adamw_step equals the same model trained by torch autograd + AdamW."""
    g, x, y, dims = S.config1()
    n = 300
    gs = S.build_graph(n, "uniform", 0, seed=2, permute=False, exact_pairs=1200)
    a, a_t = gs.torch_csr().double(), gs.torch_csr(True).double()
    dims = [12, 8, 5]
    gen = torch.Generator().manual_seed(0)
    x0 = torch.randn(n, dims[0], generator=gen, dtype=torch.float64)
    labels = torch.randint(0, 5, (n,), generator=gen)
    ws = [w.double() for w in S.glorot_weights(dims, seed=1)]
    losses, xf, wf = po.train_epochs(x0, ws, dims, [(a, a_t)], labels, n, 5, epochs=4)

    xs = x0.clone().reshape(-1).requires_grad_()
    wt = [w.clone().requires_grad_() for w in ws]
    opt = torch.optim.AdamW(wt + [xs], lr=3e-3, weight_decay=0.0)
    ref_losses = []
    for _ in range(4):
        opt.zero_grad()
        h = xs.reshape(n, dims[0])
        for i, w in enumerate(wt):
            h = torch.mm(torch.sparse.mm(a, h), w.reshape(dims[i], dims[i + 1]))
            if i != len(wt) - 1:
                h = F.relu(h)
        loss = F.cross_entropy(h, labels)
        loss.backward()
        opt.step()
        ref_losses.append(float(loss))
    assert np.allclose(losses, ref_losses, atol=1e-12)
    assert torch.allclose(xf, xs.detach(), atol=1e-12)
    for a_, b_ in zip(wf, wt):
        assert torch.allclose(a_, b_.detach(), atol=1e-12)
    assert losses[-1] < losses[0]


def test_csr_pair_construction_and_block():
    """build_csr_pair follows the loader: mask, re-base, COO->CSR, transpose->CSR."""
    gen = torch.Generator().manual_seed(0)
    ei = torch.randint(0, 20, (2, 150), generator=gen)
    ei = torch.unique(ei, dim=1)
    w = torch.rand(ei.shape[1], generator=gen)
    a, a_t = po.build_csr_pair(ei, w, (20, 20), row_range=(5, 15), col_range=(0, 10))
    dense = torch.zeros(20, 20)
    dense[ei[0], ei[1]] = w
    assert torch.equal(a.to_dense(), dense[5:15, 0:10])
    assert torch.equal(a_t.to_dense(), dense[5:15, 0:10].t())
    assert po.pad_dimension(10, 4) == 12 and po.pad_dimension(12, 4) == 12 and po.pad_dimension(7, 2, 3) == 12


def test_oracle_reproduces_committed_config1_fixture():
    """Drift guard: the oracle (and the synthetic generator feeding it) still gives the committed result."""
    import importlib.util
    import json
    import os

    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_config1_golden", os.path.join(here, "make_config1_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    want = json.load(open(os.path.join(here, "config1_golden.json")))
    got = mod.compute()
    for key in ("nnz", "col_checksum", "x_ones", "label_histogram"):
        assert got[key] == want[key], key
    assert abs(got["val_sum"] - want["val_sum"]) <= 1e-9 * abs(want["val_sum"])
    assert np.allclose(got["losses_fp64"], want["losses_fp64"], rtol=1e-10, atol=0)
    assert np.allclose(got["final_weight_abs_sum"], want["final_weight_abs_sum"], rtol=1e-9)
    assert abs(got["logits_epoch0_abs_sum"] - want["logits_epoch0_abs_sum"]) <= 1e-9 * want["logits_epoch0_abs_sum"]
    assert want["losses_fp64"][-1] < want["losses_fp64"][0]


# ---- vertex permutation and the 2-D partition files ----
def _raw_graph(n=83, pairs=500, seed=11):
    g = torch.Generator().manual_seed(seed)
    ei = torch.randint(0, n, (2, pairs), generator=g)
    w = torch.rand(pairs, generator=g) + 0.1
    ei_n, w_n = po.gcn_norm(ei, n, w)
    coo = torch.sparse_coo_tensor(ei_n, w_n, (n, n)).coalesce()  # distinct entries, so dense forms are comparable
    return coo.indices(), coo.values(), g


def test_permutation_by_sparse_products_equals_index_maps():
    n = 83
    ei, w, g = _raw_graph(n)
    x = torch.randn(n, 10, generator=g)
    y = torch.randint(0, 5, (n,), generator=g)
    perm, perm2 = torch.randperm(n, generator=g), torch.randperm(n, generator=g)
    dense = torch.sparse_coo_tensor(ei, w, (n, n)).to_dense()
    out = po.permute_graph(ei, w, x, y, perm, perm2)
    d1 = torch.sparse_coo_tensor(out["edge_index"], out["edge_weight"], (n, n)).to_dense()
    d2 = torch.sparse_coo_tensor(out["edge_index_2"], out["edge_weight_2"], (n, n)).to_dense()
    assert torch.equal(d1, dense[perm][:, perm2])  # entry (i, j) of the result is entry (perm[i], perm2[j])
    assert torch.equal(d2, dense[perm2][:, perm])
    assert torch.equal(out["x"], x[perm2]) and torch.equal(out["y"], y[perm]) and torch.equal(out["y_2"], y[perm2])
    rows = out["edge_index"][0]
    assert (rows[1:] >= rows[:-1]).all()  # rows in order; the sparse product leaves the columns of a row unsorted
    assert torch.unique(rows * n + out["edge_index"][1]).numel() == rows.numel()  # no duplicates
    # a layer is equivariant: (P A P2^T)(P2 H) = P (A H)
    h = torch.randn(n, 4, generator=g, dtype=torch.float64)
    assert torch.allclose(d1.double() @ h[perm2], (dense.double() @ h)[perm], atol=1e-12)
    # single permutation and the directed case (the transpose is what gets permuted)
    single = po.permute_graph(ei, w, x, y, perm)
    ds = torch.sparse_coo_tensor(single["edge_index"], single["edge_weight"], (n, n)).to_dense()
    assert torch.equal(ds, dense[perm][:, perm]) and torch.equal(single["x"], x[perm])
    dd = po.permute_graph(ei, w, x, y, perm, perm2, directed=True)
    assert torch.equal(torch.sparse_coo_tensor(dd["edge_index"], dd["edge_weight"], (n, n)).to_dense(), dense.t()[perm][:, perm2])


@pytest.mark.parametrize("parts", [1, 2, 3, 5])
@pytest.mark.parametrize("layers,num_gpus,ranks", [(3, (1, 1, 1), (0, 0, 0)), (3, (2, 2, 2), (1, 0, 1)), (4, (2, 3, 1), (1, 2, 0)),
                                                   (2, (1, 2, 4), (0, 1, 3)), (6, (3, 2, 2), (2, 1, 1))])
def test_partition_files_and_loader_restatement_vs_dense_slicing(tmp_path, parts, layers, num_gpus, ranks):
    """Files written by the product's partition writer (host code), read back by the oracle's restatement of the
    loader; both pinned by slicing zero-padded dense matrices."""
    from plexus_amd.utils import dataset as D

    n, f, classes = 83, 10, 5
    ei, w, g = _raw_graph(n)
    x = torch.randn(n, f, generator=g)
    y = torch.randint(0, classes, (n,), generator=g)
    perm, perm2 = torch.randperm(n, generator=g), torch.randperm(n, generator=g)
    pg = po.permute_graph(ei, w, x, y, perm, perm2)
    graph = D.ProcessedGraph(pg["edge_index"], pg["edge_weight"], pg["x"], pg["y"], classes, pg["edge_index_2"], pg["edge_weight_2"], pg["y_2"])
    D.partition_graph_2d(graph, parts, str(tmp_path))
    # layout: exactly the files the reference's loader opens
    import os
    assert sorted(os.listdir(tmp_path)) == ["edge_index", "input_features", "metadata.pt", "output_labels"]
    assert sorted(os.listdir(tmp_path / "edge_index" / "1")) == sorted("%d_%d.pt" % (i, j) for i in range(parts) for j in range(parts))
    assert torch.load(tmp_path / "metadata.pt", weights_only=True) == (n, f, classes)
    e00, w00 = torch.load(tmp_path / "edge_index" / "0" / "0_0.pt", weights_only=True)
    assert e00.dtype == torch.int64 and e00.shape[0] == 2 and w00.dtype == torch.float32
    total = sum(torch.load(tmp_path / "edge_index" / "0" / ("%d_%d.pt" % (i, j)), weights_only=True)[1].numel()
                for i in range(parts) for j in range(parts))
    assert total == graph.edge_weight.numel()  # every edge lands in exactly one file

    shards, feats, labels, nn, nf, nc = po.load_partitioned(str(tmp_path), layers, num_gpus, ranks)
    assert (nn, nf, nc) == (n, f, classes)
    big = 2 * n + 16
    dense = [torch.zeros(big, big), torch.zeros(big, big)]
    dense[0][:n, :n] = torch.sparse_coo_tensor(pg["edge_index"], pg["edge_weight"], (n, n)).to_dense()
    dense[1][:n, :n] = torch.sparse_coo_tensor(pg["edge_index_2"], pg["edge_weight_2"], (n, n)).to_dense()
    groups = [(0, 1), (2, 0), (1, 2)]
    assert len(shards) == min(6, layers)
    for layer, (a, at) in enumerate(shards):
        g1, g2 = groups[layer % 3]
        s1 = po.pad_dimension(n, num_gpus[g1]) // num_gpus[g1]
        s2 = po.pad_dimension(n, num_gpus[g2]) // num_gpus[g2]
        want = dense[layer % 2][ranks[g1] * s1:(ranks[g1] + 1) * s1, ranks[g2] * s2:(ranks[g2] + 1) * s2]
        assert tuple(a.shape) == (s1, s2) and torch.equal(a.to_dense(), want) and torch.equal(at.to_dense(), want.t())
    # features: rows of the x group, columns of the y group (padded to y * z), flattened and cut by the depth group
    ns = po.pad_dimension(n, num_gpus[1]) // num_gpus[1]
    fs = po.pad_dimension(f, num_gpus[2], num_gpus[0]) // num_gpus[2]
    xp = torch.zeros(big, big)
    xp[:n, :f] = pg["x"]
    slab = xp[ranks[1] * ns:(ranks[1] + 1) * ns, ranks[2] * fs:(ranks[2] + 1) * fs].reshape(-1)
    ds = slab.numel() // num_gpus[0]
    assert slab.numel() % num_gpus[0] == 0 and torch.equal(feats, slab[ranks[0] * ds:(ranks[0] + 1) * ds])
    # labels: the group that splits the rows of the last layer's output; second labels for an even layer count
    lg = {1: 0, 2: 2, 0: 1}[layers % 3]
    ls = po.pad_dimension(n, num_gpus[lg]) // num_gpus[lg]
    yp = torch.zeros(big, dtype=torch.int64)
    yp[:n] = pg["y_2"] if layers % 2 == 0 else pg["y"]
    assert torch.equal(labels, yp[ranks[lg] * ls:(ranks[lg] + 1) * ls])


# ---- the bf16-storage restatement (OracleNetBf16): pinned against OracleNet and against autograd ----
def _ring_graph(n, dtype):
    """Row i holds columns i-1, i, i+2 (mod n) with value 1: three entries per row and per column, not symmetric."""
    rows = torch.arange(n).repeat_interleave(3)
    cols = (rows + torch.tensor([-1, 0, 2]).repeat(n)) % n
    a = torch.sparse_coo_tensor(torch.stack([rows, cols]), torch.ones(3 * n, dtype=dtype), (n, n)).to_sparse_csr()
    return a, a.transpose(0, 1).to_sparse_csr()


def test_bf16_oracle_equals_fp32_oracle_when_rounding_is_the_identity():
    """Small-integer operands: every stored tensor is exactly representable in bf16, every rounding is the identity and
    there is no dropout, so the bf16 restatement must give OracleNet's numbers bit for bit (forward, grad_x, grad_w).
    A transposed weight, a mask taken from the wrong tensor or a misplaced product changes an integer somewhere."""
    n, dims = 40, [5, 4, 3]
    gen = torch.Generator().manual_seed(4)
    for dtype in (torch.float32, torch.float64):
        a, a_t = _ring_graph(n, dtype)
        x = torch.randint(-1, 2, (n * dims[0],), generator=gen).to(dtype)
        ws = [torch.randint(-1, 2, (dims[i] * dims[i + 1],), generator=gen).to(dtype) for i in range(2)]
        g_logits = torch.randint(-1, 2, (n, dims[-1]), generator=gen).to(dtype)
        ref = po.OracleNet(ws, dims)
        out_ref = ref.forward(x, [(a, a_t)])
        gx_ref, gw_ref = ref.backward(g_logits)
        # precondition: everything the bf16 path stores survives the rounding unchanged
        for agg, _, _, pre, _ in ref._saved:
            assert torch.equal(po.rb(agg), agg) and torch.equal(po.rb(pre), pre)
        assert torch.equal(po.rb(gx_ref), gx_ref) and (ref._saved[0][3] > 0).any() and (ref._saved[0][3] < 0).any()
        net = po.OracleNetBf16(ws, dims, dropout_p=0.0)
        out = net.forward(x, [(a, a_t)])
        gx, gw = net.backward(g_logits)
        assert torch.equal(out, out_ref)
        assert torch.equal(gx.reshape(-1), gx_ref.reshape(-1))
        for u, v in zip(gw, gw_ref):
            assert torch.equal(u, v) and u.abs().sum() > 0


class _RoundBoth(torch.autograd.Function):
    """bf16 rounding of a stored tensor: the value is rounded on the way forward and its gradient on the way back."""

    @staticmethod
    def forward(ctx, t):
        return po.rb(t)

    @staticmethod
    def backward(ctx, g):
        return po.rb(g)


def _bf16_forward_autograd(x, ws, dims, a, p, keeps):
    """The forward of OracleNetBf16 as a differentiable graph: weights rounded straight-through, stored activations
    through _RoundBoth, the dropout keep-mask a constant factor."""
    h = _RoundBoth.apply(x)
    for i, w in enumerate(ws):
        w2 = w.reshape(dims[i], dims[i + 1])
        w_st = w2 + (po.rb(w2) - w2).detach()  # value rb(w), gradient passed to w unchanged
        agg = _RoundBoth.apply(torch.sparse.mm(a, h.reshape(a.shape[1], dims[i])))
        out = torch.mm(agg, w_st)
        if i != len(ws) - 1:
            out = F.relu(out)
            if p > 0:
                out = out * keeps[i] / (1.0 - p)
        h = _RoundBoth.apply(out)
    return h


@pytest.mark.parametrize("p", [0.0, 0.5])
def test_bf16_oracle_backward_equals_autograd_over_its_forward(p):
    """Hand backward of OracleNetBf16 == torch.autograd over the same forward (fp64; power-of-two dropout scale, so both
    orders of applying it give the same bits).  Fails if 1/(1-p) is missing or doubled in grad_w or grad_agg, if the
    mask comes from a tensor that ignores dropout, or if a weight is transposed."""
    n, dims, seed = 70, [9, 7, 6, 4], 5
    a = small_graph(n=n, pairs=350, seed=21).double()
    a_t = a.transpose(0, 1).to_sparse_csr()
    gen = torch.Generator().manual_seed(8)
    x = torch.randn(n * dims[0], generator=gen, dtype=torch.float64)
    ws = [torch.randn(dims[i] * dims[i + 1], generator=gen, dtype=torch.float64) for i in range(3)]
    g_logits = torch.randn(n, dims[-1], generator=gen, dtype=torch.float64)
    offsets = [11, 12, 13]
    keeps = [torch.from_numpy(po.dropout_keep_mask(n * dims[i + 1], seed, offsets[i], p).reshape(n, dims[i + 1])).double()
             for i in range(2)]

    net = po.OracleNetBf16(ws, dims, dropout_p=p, seed=seed)
    out = net.forward(x, [(a, a_t)], offsets=offsets)
    gx, gw = net.backward(g_logits)

    xs = x.clone().requires_grad_()
    wt = [w.clone().requires_grad_() for w in ws]
    out_ag = _bf16_forward_autograd(xs, wt, dims, a, p, keeps)
    assert torch.equal(out, out_ag.detach())
    grads = torch.autograd.grad(out_ag, [xs] + wt, g_logits)
    scale = lambda t: t.abs().max()
    assert (gx.reshape(-1) - grads[0]).abs().max() <= 1e-13 * scale(grads[0])
    for u, v in zip(gw, grads[1:]):
        assert (u - v).abs().max() <= 1e-13 * scale(v) and scale(v) > 0
    if p > 0:  # the mask really dropped something, and dropped units carry no gradient
        assert 0.3 < keeps[0].mean() < 0.7
        assert (net._saved[0][2][keeps[0] == 0] == 0).all()


def test_bf16_oracle_dropout_scale_appears_once():
    """One hidden layer, p = 0.5: grad_w of the hidden layer and the gradient handed to the aggregation are exactly
    1/(1-p) = 2 times what the same network gives when the kept units are selected by a 0/1 mask without rescaling
    (computed here from the saved tensors with plain products)."""
    n, dims, p, seed = 50, [6, 5, 3], 0.5, 2
    a = small_graph(n=n, pairs=260, seed=31).double()
    a_t = a.transpose(0, 1).to_sparse_csr()
    gen = torch.Generator().manual_seed(9)
    x = torch.randn(n * dims[0], generator=gen, dtype=torch.float64)
    ws = [torch.randn(dims[i] * dims[i + 1], generator=gen, dtype=torch.float64) for i in range(2)]
    g_logits = torch.randn(n, dims[-1], generator=gen, dtype=torch.float64)
    net = po.OracleNetBf16(ws, dims, dropout_p=p, seed=seed)
    net.forward(x, [(a, a_t)], offsets=[3, 4])
    gx, gw = net.backward(g_logits)
    keep = torch.from_numpy(po.dropout_keep_mask(n * dims[1], seed, 3, p).reshape(n, dims[1])).double()
    agg0, _, out0, _ = net._saved[0]
    agg1 = net._saved[1][0]
    w0, w1 = (po.rb(w.reshape(dims[i], dims[i + 1])) for i, w in enumerate(ws))
    pre0 = agg0 @ w0
    assert torch.equal(out0, po.rb(F.relu(pre0) * keep * 2.0))
    g1 = po.rb(g_logits)
    assert torch.allclose(gw[1], (agg1.t() @ g1).reshape(-1), rtol=1e-13, atol=0)  # last layer: no scale at all
    g_h = po.rb(a_t.to_dense() @ po.rb(g1 @ w1.t())) * ((pre0 > 0).double() * keep)  # unscaled, 0/1 selection
    assert torch.allclose(gw[0], 2.0 * (agg0.t() @ g_h).reshape(-1), rtol=1e-12, atol=1e-14)
    assert torch.allclose(gx.reshape(n, dims[0]), po.rb(a_t.to_dense() @ po.rb(2.0 * (g_h @ w0.t()))), rtol=1e-12, atol=1e-14)


def test_bf16_epoch_loop_matches_autograd_training():
    """train_epochs_bf16 == the same bf16-storage model (rounded values, rounded stored gradients, constant dropout masks)
    trained by torch autograd + F.cross_entropy + torch.optim.AdamW, in fp64."""
    n, dims, p, seed, epochs = 70, [9, 7, 6, 4], 0.5, 5, 3
    a = small_graph(n=n, pairs=350, seed=21).double()
    a_t = a.transpose(0, 1).to_sparse_csr()
    gen = torch.Generator().manual_seed(8)
    x0 = torch.randn(n * dims[0], generator=gen, dtype=torch.float64)
    ws = [torch.randn(dims[i] * dims[i + 1], generator=gen, dtype=torch.float64) * 0.3 for i in range(3)]
    labels = torch.randint(0, dims[-1], (n,), generator=gen)
    offs = lambda e: [i + 64 * e for i in range(3)]
    losses, xf, wf = po.train_epochs_bf16(x0, ws, dims, [(a, a_t)], labels, n, dims[-1], epochs=epochs, dropout_p=p, seed=seed,
                                          offsets_of_epoch=offs)
    xs = x0.clone().requires_grad_()
    wt = [w.clone().requires_grad_() for w in ws]
    opt = torch.optim.AdamW(wt + [xs], lr=3e-3, weight_decay=0.0)
    ref_losses = []
    for e in range(epochs):
        keeps = [torch.from_numpy(po.dropout_keep_mask(n * dims[i + 1], seed, offs(e)[i], p).reshape(n, dims[i + 1])).double()
                 for i in range(2)]
        opt.zero_grad()
        loss = F.cross_entropy(_bf16_forward_autograd(xs, wt, dims, a, p, keeps), labels)
        loss.backward()
        opt.step()
        ref_losses.append(float(loss.detach()))
    assert np.allclose(losses, ref_losses, rtol=1e-12, atol=0)
    assert torch.allclose(xf, xs.detach(), rtol=0, atol=1e-12)
    for u_, v_ in zip(wf, wt):
        assert torch.allclose(u_, v_.detach(), rtol=0, atol=1e-12)
    assert losses[0] != losses[1]


@pytest.mark.parametrize("p", [0.5, 0.25])
def test_fp32_oracle_with_dropout_backward_equals_autograd_over_its_forward(p):
    """OracleNet with dropout after the ReLU: the hand backward == torch.autograd over the plain-operator forward with the
    keep masks as constant factors (fp64).  Fails if 1/(1-p) is missing or doubled in grad_w or in the gradient handed to
    the aggregation, if dropped units keep a gradient, or if the last layer is dropped too."""
    n, dims, seed = 70, [9, 7, 6, 4], 5
    a = small_graph(n=n, pairs=350, seed=21).double()
    a_t = a.transpose(0, 1).to_sparse_csr()
    gen = torch.Generator().manual_seed(8)
    x = torch.randn(n * dims[0], generator=gen, dtype=torch.float64)
    ws = [torch.randn(dims[i] * dims[i + 1], generator=gen, dtype=torch.float64) for i in range(3)]
    g_logits = torch.randn(n, dims[-1], generator=gen, dtype=torch.float64)
    offsets = [11, 12, 13]
    keeps = [torch.from_numpy(po.dropout_keep_mask(n * dims[i + 1], seed, offsets[i], p).reshape(n, dims[i + 1])).double()
             for i in range(2)]
    net = po.OracleNet(ws, dims, dropout_p=p, seed=seed)
    out = net.forward(x, [(a, a_t)], offsets=offsets)
    gx, gw = net.backward(g_logits)

    xs = x.clone().requires_grad_()
    wt = [w.clone().requires_grad_() for w in ws]
    h = xs
    for i, w in enumerate(wt):
        h = torch.mm(torch.sparse.mm(a, h.reshape(n, dims[i])), w.reshape(dims[i], dims[i + 1]))
        if i != 2:
            h = F.dropout(F.relu(h), 0.0) * keeps[i] / (1.0 - p)
    assert torch.allclose(out, h.detach(), rtol=1e-14, atol=0)
    grads = torch.autograd.grad(h, [xs] + wt, g_logits)
    scale = lambda t: t.abs().max()
    assert (gx.reshape(-1) - grads[0]).abs().max() <= 1e-13 * scale(grads[0])
    for u, v in zip(gw, grads[1:]):
        assert (u - v).abs().max() <= 1e-13 * scale(v) and scale(v) > 0
    assert abs(float(keeps[0].mean()) - (1.0 - p)) < 0.12  # the mask drops about p of the units
    assert (net._saved[0][3][keeps[0] == 0] != 0).any()  # ... units that were alive before it
    # without dropout the class is what it was: same numbers as a net built without the arguments
    plain, plain0 = po.OracleNet(ws, dims), po.OracleNet(ws, dims, dropout_p=0.0, seed=3)
    assert torch.equal(plain.forward(x, [(a, a_t)]), plain0.forward(x, [(a, a_t)], offsets=offsets))
