"""Graph preprocessing and the partition-file loader on the GPU against the CPU oracle.

Index work (permutations, edge lists, CSR structure, labels, feature slabs) must be bit-exact; normalised
weights are fp32 and held to max|x - ref| / max|ref| <= 1e-5."""
import pytest
import torch

from conftest import FP32_TOL, rel_err
from oracle import plexus_oracle as po
from plexus_amd import ops
from plexus_amd.utils import dataset as D
from plexus_amd.utils.dataloader import DataLoader

pytestmark = pytest.mark.gpu
DEV = "cuda"


def say(msg):
    print("[case] " + msg, flush=True)


def raw_edges(n, pairs, seed, loops=True, symmetric=False):
    g = torch.Generator().manual_seed(seed)
    ei = torch.randint(0, n, (2, pairs), generator=g)
    if symmetric:
        ei = torch.cat([ei, ei.flip(0)], dim=1)
    if loops:  # a few existing self loops with their own weights
        k = torch.randint(0, n, (5,), generator=g)
        ei = torch.cat([ei, torch.stack([k, k])], dim=1)
    w = torch.rand(ei.shape[1], generator=g) + 0.1
    if symmetric:
        w[pairs:2 * pairs] = w[:pairs]
    # distinct pairs only: the weight an existing self loop keeps is then unambiguous
    coo = torch.sparse_coo_tensor(ei, w, (n, n)).coalesce()
    return coo.indices(), coo.values(), g


def sorted_edges(ei, w, n):
    order = torch.argsort(ei[0] * n + ei[1])
    return ei[:, order], w[order]


def test_permutation_kernels_exact():
    say("invert_permutation / relabel_edges / csr_to_edges")
    g = torch.Generator().manual_seed(5)
    n = 100003
    perm = torch.randperm(n, generator=g)
    inv = ops.invert_permutation(perm.to(DEV)).cpu()
    assert torch.equal(inv[perm], torch.arange(n)) and torch.equal(perm[inv], torch.arange(n))
    ei = torch.randint(0, n, (2, 300001), generator=g)
    ei[0, 7] = -3
    ei[1, 9] = n  # ids outside the maps come back as -1
    perm2 = torch.randperm(n, generator=g)
    out = ops.relabel_edges(ei.to(DEV), perm.to(DEV), perm2.to(DEV)).cpu()
    want = torch.stack([perm[ei[0].clamp(0, n - 1)], perm2[ei[1].clamp(0, n - 1)]])
    want[0, 7] = -1
    want[1, 9] = -1
    assert torch.equal(out, want)
    # CSR -> edge list, with empty rows and one long row
    counts = torch.randint(0, 6, (5000,), generator=g)
    counts[::17] = 0
    counts[1234] = 40000
    rowptr = torch.zeros(5001, dtype=torch.int64)
    rowptr[1:] = torch.cumsum(counts, 0)
    nnz = int(rowptr[-1])
    col = torch.randint(0, 5000, (nnz,), generator=g)
    a = ops.CsrMatrix(rowptr.to(DEV), col.to(DEV), torch.ones(nnz, device=DEV), (5000, 5000))
    e, w = ops.csr_to_edges(a)
    assert torch.equal(e[0].cpu(), torch.repeat_interleave(torch.arange(5000), counts)) and torch.equal(e[1].cpu(), col)
    empty = ops.CsrMatrix(torch.zeros(4, dtype=torch.int64, device=DEV), torch.zeros(0, dtype=torch.int64, device=DEV),
                          torch.zeros(0, device=DEV), (3, 3))
    assert ops.csr_to_edges(empty)[0].shape == (2, 0)


@pytest.mark.parametrize("directed", [False, True])
def test_gcn_norm_from_edge_list(directed):
    say("dataset.gcn_norm directed=%s" % directed)
    n = 3000
    ei, w, _ = raw_edges(n, 20000, seed=1, symmetric=not directed)
    a = D.gcn_norm(ei.to(DEV), w.to(DEV), n, directed=directed)
    ref_ei, ref_w = po.gcn_norm(ei, n, w)
    if directed:
        ref_ei = ref_ei.flip(0)
    ref_ei, ref_w = sorted_edges(ref_ei, ref_w, n)
    got_ei, got_w = ops.csr_to_edges(a)
    assert torch.equal(got_ei.cpu(), ref_ei)
    assert rel_err(got_w.cpu(), ref_w) <= FP32_TOL
    ref64 = po.gcn_norm(ei, n, w, dtype=torch.float64)
    assert rel_err(got_w.cpu(), sorted_edges(ref64[0].flip(0) if directed else ref64[0], ref64[1], n)[1]) <= FP32_TOL


@pytest.mark.parametrize("directed", [False, True])
def test_gcn_norm_with_duplicates_loops_isolated_vertices_and_strays(directed):
    """Raw (uncoalesced) edge lists: duplicate edges and duplicate self loops are summed, isolated vertices get their
    loop, edges that name a vertex outside the graph are dropped, and a hub vertex collects a long column."""
    say("dataset.gcn_norm raw edge list directed=%s" % directed)
    n = 4000
    g = torch.Generator().manual_seed(11)
    ei = torch.randint(0, n - 50, (2, 30000), generator=g)  # the last 50 vertices stay isolated
    hub = torch.stack([torch.randint(0, n - 50, (6000,), generator=g), torch.full((6000,), 17)])  # in-degree ~6000
    dup = ei[:, :500]  # every one of these edges twice more
    loops = torch.tensor([[3, 3, 3, 99], [3, 3, 3, 99]])  # vertex 3 has three loops, vertex 99 one
    ei = torch.cat([ei, hub, dup, loops, dup], dim=1)
    ei = ei[:, torch.randperm(ei.shape[1], generator=g)]
    w = torch.rand(ei.shape[1], generator=g) + 0.1
    ref_ei, ref_w = po.gcn_norm(ei, n, w)
    ref64 = po.gcn_norm(ei, n, w, dtype=torch.float64)[1]
    if directed:
        ref_ei = ref_ei.flip(0)
    coo = torch.sparse_coo_tensor(ref_ei, ref_w, (n, n)).coalesce()  # duplicates summed, sorted by (row, col)
    coo64 = torch.sparse_coo_tensor(ref_ei, ref64, (n, n)).coalesce()
    stray = torch.tensor([[-1, 5, n, 2], [4, n + 3, 1, -7]])
    ei_dev = torch.cat([ei[:, :100], stray, ei[:, 100:]], dim=1).to(DEV)
    w_dev = torch.cat([w[:100], torch.ones(4), w[100:]]).to(DEV)
    a = D.gcn_norm(ei_dev, w_dev, n, directed=directed)
    got_ei, got_w = ops.csr_to_edges(a)
    assert a.nnz == coo.indices().shape[1] and int(a.rowptr[-1]) == a.nnz
    assert torch.equal(got_ei.cpu(), coo.indices())
    assert rel_err(got_w.cpu(), coo.values()) <= FP32_TOL and rel_err(got_w.cpu(), coo64.values()) <= FP32_TOL
    # unit weights when none are given; integers, so the sums are exact and the values follow from the degrees alone
    b = D.gcn_norm(ei.to(DEV), None, n, directed=directed)
    ref1_ei, ref1_w = po.gcn_norm(ei, n, None)
    coo1 = torch.sparse_coo_tensor(ref1_ei.flip(0) if directed else ref1_ei, ref1_w, (n, n)).coalesce()
    b_ei, b_w = ops.csr_to_edges(b)
    assert torch.equal(b_ei.cpu(), coo1.indices()) and rel_err(b_w.cpu(), coo1.values()) <= FP32_TOL


def test_gcn_norm_of_a_graph_without_edges_is_the_identity():
    say("dataset.gcn_norm without edges")
    a = D.gcn_norm(torch.zeros((2, 0), dtype=torch.int64, device=DEV), None, 7)
    assert torch.equal(a.rowptr.cpu(), torch.arange(8, dtype=torch.int32)) and torch.equal(a.col.cpu(), torch.arange(7, dtype=torch.int32))
    assert torch.equal(a.val.cpu(), torch.ones(7))
    h = torch.randn(7, 5, device=DEV)
    assert torch.equal(ops.spmm(a, h), h)  # and the deferred plan is built by the first product


def test_csr_permute_matches_the_sparse_products_and_refuses_a_non_permutation():
    say("ops.csr_permute")
    n, k = 3000, 2500  # rectangular, with empty rows and one hub row
    g = torch.Generator().manual_seed(12)
    counts = torch.randint(0, 9, (n,), generator=g)
    counts[::13] = 0
    counts[77] = 2400
    rows = torch.repeat_interleave(torch.arange(n), counts)
    cols = torch.cat([torch.randperm(k, generator=g)[:c] for c in counts.tolist()])
    vals = torch.rand(rows.numel(), generator=g)
    dense = torch.zeros(n, k)
    dense[rows, cols] = vals
    a = ops.csr_from_edges(torch.stack([rows, cols]).to(DEV), vals.to(DEV), (n, k))
    p_r, p_c = torch.randperm(n, generator=g), torch.randperm(k, generator=g)
    got = ops.csr_permute(a, p_r.to(DEV), p_c.to(DEV))
    want = dense[p_r][:, p_c].to_sparse_csr()  # new[i, j] = old[perm_rows[i], perm_cols[j]]
    assert torch.equal(got.rowptr.cpu().long(), want.crow_indices()) and torch.equal(got.col.cpu().long(), want.col_indices())
    assert torch.equal(got.val.cpu(), want.values())  # values only move
    h = torch.randn(k, 9, device=DEV)
    assert rel_err(ops.spmm(got, h).cpu(), (dense[p_r][:, p_c].double() @ h.cpu().double()).float()) <= FP32_TOL
    a_t = ops.csr_transpose(a)
    again = ops.csr_permute(a, p_r.to(DEV), p_c.to(DEV), a_t=a_t)  # from a transpose built by the caller
    assert torch.equal(again.rowptr, got.rowptr) and torch.equal(again.col, got.col) and torch.equal(again.val, got.val)
    twice = p_r.clone()
    twice[5] = twice[6]  # one row twice, another never
    with pytest.raises(RuntimeError, match="outside"):
        ops.csr_permute(a, twice.to(DEV), p_c.to(DEV), a_t=a_t)
    stray = p_r.clone()
    stray[3] = n
    with pytest.raises(RuntimeError, match="outside"):
        ops.csr_permute(a, stray.to(DEV), p_c.to(DEV), a_t=a_t)
    col_counts = torch.bincount(cols, minlength=k)
    twice = p_c.clone()
    twice[5] = p_c[int((col_counts[p_c] != col_counts[p_c[5]]).nonzero()[0])]  # a column of another length in place of one
    with pytest.raises(RuntimeError, match="not a permutation"):
        ops.csr_permute(a, p_r.to(DEV), twice.to(DEV), a_t=a_t)
    with pytest.raises(ValueError):
        ops.csr_permute(a, p_r.to(DEV), p_c.to(DEV), a_t=a)  # not the transpose's shape
    with pytest.raises(ValueError):
        ops.csr_permute(a, p_r[:-1].to(DEV), p_c.to(DEV))
    empty = ops.CsrMatrix(torch.zeros(5, dtype=torch.int64, device=DEV), torch.zeros(0, dtype=torch.int64, device=DEV),
                          torch.zeros(0, device=DEV), (4, 4))
    e = ops.csr_permute(empty, torch.randperm(4).to(DEV), torch.randperm(4).to(DEV))
    assert e.nnz == 0 and torch.equal(e.rowptr.cpu(), torch.zeros(5, dtype=torch.int32))


@pytest.mark.parametrize("double_perm,directed", [(True, False), (False, False), (True, True)])
def test_preprocess_graph_matches_sparse_product_permutation(double_perm, directed):
    say("preprocess_graph double_perm=%s directed=%s" % (double_perm, directed))
    n, f, classes = 2000, 24, 7
    ei, w, g = raw_edges(n, 15000, seed=2, symmetric=not directed)
    x = torch.randn(n, f, generator=g)
    y = torch.randint(0, classes, (n,), generator=g)
    perm, perm2 = torch.randperm(n, generator=g), torch.randperm(n, generator=g)
    got = D.preprocess_graph(ei.to(DEV), w.to(DEV), x.to(DEV), y.to(DEV), classes, double_perm=double_perm, directed=directed,
                             perm=perm, perm2=perm2)
    nei, nw = po.gcn_norm(ei, n, w)
    ref = po.permute_graph(nei, nw, x, y, perm, perm2 if double_perm else None, directed=directed)
    r_ei, r_w = sorted_edges(ref["edge_index"], ref["edge_weight"], n)
    assert torch.equal(got.edge_index.cpu(), r_ei) and rel_err(got.edge_weight.cpu(), r_w) <= FP32_TOL
    assert torch.equal(got.x.cpu(), ref["x"]) and torch.equal(got.y.cpu(), ref["y"])
    assert got.double_perm == double_perm
    if double_perm:
        r_ei2, r_w2 = sorted_edges(ref["edge_index_2"], ref["edge_weight_2"], n)
        assert torch.equal(got.edge_index_2.cpu(), r_ei2) and rel_err(got.edge_weight_2.cpu(), r_w2) <= FP32_TOL
        assert torch.equal(got.y_2.cpu(), ref["y_2"])


def test_unsupervised_features_and_degree_bucket_labels():
    say("preprocess_graph without features or labels")
    n, classes = 1000, 6
    ei, w, _ = raw_edges(n, 6000, seed=4, symmetric=True)
    got = D.preprocess_graph(ei.to(DEV), None, None, None, classes, double_perm=False, num_features=16,
                             generator=torch.Generator().manual_seed(0), perm=torch.arange(n), num_nodes=n)
    assert got.x.shape == (n, 16) and (got.x.sum(1) <= 1.0 + 1e-6).all()  # row sums clamped at 1 from below before dividing
    counts = torch.bincount(po.gcn_norm(ei, n)[0][0], minlength=n)
    y = got.y.cpu()
    sizes = torch.bincount(y, minlength=classes)
    assert sizes.max() - sizes.min() <= 1 and (sizes[:-1] >= sizes[1:]).all()  # numpy.array_split sizes
    for c in range(classes - 1):  # buckets are ordered by degree
        assert counts[y == c].max() <= counts[y == c + 1].min()


@pytest.mark.parametrize("parts", [1, 3])
@pytest.mark.parametrize("layers,grid,ranks", [(3, (1, 1, 1), (0, 0, 0)), (4, (1, 1, 1), (0, 0, 0)), (3, (2, 2, 2), (0, 1, 1)),
                                               (5, (3, 1, 2), (2, 0, 1))])
def test_partition_files_loader_matches_host_loader(tmp_path, parts, layers, grid, ranks):
    say("partition_graph_2d + DataLoader parts=%d layers=%d grid=%s ranks=%s" % (parts, layers, grid, ranks))
    n, f, classes = 1500, 20, 5
    ei, w, g = raw_edges(n, 12000, seed=3, symmetric=True)
    x = torch.randn(n, f, generator=g)
    y = torch.randint(0, classes, (n,), generator=g)
    graph = D.preprocess_graph(ei.to(DEV), w.to(DEV), x.to(DEV), y.to(DEV), classes, generator=g)
    D.partition_graph_2d(graph, parts, str(tmp_path))
    shards, feats, labels, nn, nf, nc = DataLoader(str(tmp_path), layers, grid=grid, ranks=ranks).load()
    # the host loader takes the groups in the reference's (depth, row, column) order
    r_shards, r_feats, r_labels, rn, rf, rc = po.load_partitioned(str(tmp_path), layers, (grid[2], grid[0], grid[1]),
                                                                  (ranks[2], ranks[0], ranks[1]))
    assert (nn, nf, nc) == (rn, rf, rc) == (n, f, classes)
    assert len(shards) == len(r_shards) == min(6, layers)
    for (a, at), (ra, rat) in zip(shards, r_shards):
        for mine, ref in ((a, ra), (at, rat)):
            assert mine.shape == tuple(ref.shape)
            assert torch.equal(mine.rowptr.cpu().long(), ref.crow_indices()) and torch.equal(mine.col.cpu().long(), ref.col_indices())
            assert torch.equal(mine.val.cpu(), ref.values())
    assert feats.requires_grad and torch.equal(feats.detach().cpu(), r_feats)
    assert labels.dtype == torch.int64 and torch.equal(labels.cpu(), r_labels)


def test_loaded_graph_trains_and_loss_is_permutation_invariant(tmp_path):
    """Three layers on a doubly permuted, partitioned graph: same loss and weight gradients as the oracle on
    the un-permuted graph (a GCN is equivariant under vertex relabelling and the loss is a mean over vertices)."""
    say("double permutation end to end")
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.train import Net
    from plexus_amd.utils import synthetic as S

    n, classes = 1200, 6
    dims = [12, 16, 16, classes]
    ei, w, g = raw_edges(n, 9000, seed=6, symmetric=True)
    x = torch.randn(n, dims[0], generator=g)
    y = torch.randint(0, classes, (n,), generator=g)
    ws = S.glorot_weights(dims, seed=1)
    graph = D.preprocess_graph(ei.to(DEV), w.to(DEV), x.to(DEV), y.to(DEV), classes, generator=g)
    D.partition_graph_2d(graph, 2, str(tmp_path))
    shards, feats, labels, nn, nf, nc = DataLoader(str(tmp_path), 3).load()
    model = Net(3, dims[0], dims[1], dims[-1], weights=ws, fuse_relu=True)
    out = model(feats, shards)
    loss = parallel_cross_entropy(out, labels, 3, nn, nc)
    loss.backward()
    # oracle on the original vertex order
    nei, nw = po.gcn_norm(ei, n, w)
    a, at = po.build_csr_pair(nei, nw, (n, n))
    net = po.OracleNet([t.clone() for t in ws], dims)
    logits = net.forward(x.reshape(-1), [(a, at)])
    rl, sm, oh = po.cross_entropy_forward(logits, y, n, classes)
    _, gws = net.backward(po.cross_entropy_backward(sm, oh.float(), n))
    assert abs(loss.item() - rl.item()) <= FP32_TOL * abs(rl.item())
    for layer, gw in zip(model.layers, gws):
        assert rel_err(layer.weight.grad.cpu(), gw.reshape(-1)) <= 2 * FP32_TOL  # two fp32 paths in different vertex orders
