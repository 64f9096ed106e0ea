"""The hot-path entry points are stream-ordered, allocate nothing and share no state: a caller may record them into
a HIP graph, and host threads may drive different streams at once.

Forward, loss and backward of a two-layer network are captured once and replayed several times with new inputs
written into the captured buffers; eager work and synchronisations sit between the replays, and every replay is
compared bit for bit with an eager run on the same inputs (the kernels have a fixed summation order).
"""
import pytest
import torch

from plexus_amd import ops
from plexus_amd.cross_entropy import parallel_cross_entropy
from plexus_amd.train import Net
from plexus_amd.utils import synthetic as S

pytestmark = pytest.mark.gpu
DEV = "cuda"


def say(msg):
    print("[case] " + msg, flush=True)


def to_dev(g, transpose=False, seg_len=0):
    if transpose:
        return ops.CsrMatrix(g.rowptr_t.to(DEV), g.col_t.to(DEV), g.val_t.to(DEV), (g.shape[1], g.shape[0]), seg_len)
    return ops.CsrMatrix(g.rowptr.to(DEV), g.col.to(DEV), g.val.to(DEV), g.shape, seg_len)


@pytest.mark.filterwarnings("ignore:The AccumulateGrad node")  # the warm-up runs on a side stream on purpose
@pytest.mark.parametrize("association,hub", [("reference", False), ("auto", False), ("reference", True)])
def test_forward_loss_backward_replay_from_a_hip_graph(association, hub):
    say("HIP graph capture of forward + loss + backward, association=%s, hub pass=%s" % (association, hub))
    n, dims, classes = 3000, ([128, 64, 7] if hub else [40, 32, 7]), 7
    g = S.build_graph(n, "chunglu", 40000, seed=5, device="cpu", gamma=2.1)
    shards = [(to_dev(g, seg_len=64), to_dev(g, True, seg_len=64))]  # split rows: the workspace path is recorded too
    assert shards[0][0].n_long_rows > 0
    if hub:  # the longest rows go through the hub pass (its kernels, its LDS size attribute and its workspace are recorded too)
        for a in shards[0]:
            a.build_hub()
            assert a.n_hub_rows > 0
    ws = S.glorot_weights(dims, seed=3)
    model = Net(2, dims[0], dims[1], dims[2], weights=ws, fuse_relu=True, association=association)
    params = list(model.parameters())
    gen = torch.Generator().manual_seed(11)
    x = torch.randn(n * dims[0], generator=gen).to(DEV).requires_grad_()
    y = torch.randint(0, classes, (n,), generator=gen).to(DEV)

    def forward_backward():
        for p in params + [x]:
            p.grad = None
        loss = parallel_cross_entropy(model(x, shards), y, 2, n, classes)
        loss.backward()
        return loss

    # warm-up on a side stream (allocates the per-matrix workspaces outside the graph's pool)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            forward_backward()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_loss = forward_backward()
    g_grads = [p.grad for p in params + [x]]
    assert all(t is not None for t in g_grads)

    for replay in range(4):
        # new inputs, written into the buffers the graph reads
        with torch.no_grad():
            x.copy_(torch.randn(n * dims[0], generator=gen).to(DEV))
            y.copy_(torch.randint(0, classes, (n,), generator=gen).to(DEV))
            for p in params:
                p.mul_(1.0 + 0.01 * (replay + 1))
        graph.replay()
        torch.cuda.synchronize()
        got = [g_loss.clone()] + [t.clone() for t in g_grads]
        # eager work between the replays: the same step outside the graph, with its own output tensors
        e_loss = forward_backward()
        torch.cuda.synchronize()
        want = [e_loss] + [p.grad for p in params + [x]]
        for a, b in zip(got, want):
            assert a.shape == b.shape and torch.equal(a, b), "replay %d differs from the eager step" % replay
        assert torch.isfinite(got[0]).all() and got[-1].abs().max() > 0


def test_threads_on_their_own_streams_give_the_serial_result():
    """The library keeps no global state: host threads driving different streams at once, each with its own matrices
    and scratch, get what a single thread gets (ctypes releases the interpreter lock during a call)."""
    import threading

    say("four host threads, four streams")
    n, d_in, d_out = 4000, 96, 40
    jobs = []
    for i in range(4):
        g = S.build_graph(n, "chunglu", 50000, seed=20 + i, device="cpu", gamma=2.2)
        gen = torch.Generator().manual_seed(i)
        jobs.append(dict(a=to_dev(g, seg_len=128), at=to_dev(g, True, seg_len=128),
                         h=torch.randn(n, d_in, generator=gen).to(DEV), w=torch.randn(d_in, d_out, generator=gen).to(DEV),
                         y=torch.randint(0, d_out, (n,), generator=gen).to(DEV)))

    def layer(j):
        agg = ops.spmm(j["a"], j["h"])
        out = ops.gemm_nn(agg, j["w"], relu=True)
        loss, gout = ops.softmax_xent(out, j["y"], n, d_out)
        gw = ops.gemm_tn(agg, gout, mask=out)
        gh = ops.spmm(j["at"], ops.gemm_nt(gout, j["w"], mask=out))
        return [loss, gw, gh]

    serial = [[t.clone() for t in layer(j)] for j in jobs]
    torch.cuda.synchronize()
    results, errors = [None] * len(jobs), []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(5):
                    results[i] = layer(jobs[i])
            stream.synchronize()
        except Exception as e:  # surfaced in the main thread below
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
    assert not errors, errors
    torch.cuda.synchronize()
    for want, got in zip(serial, results):
        for a, b in zip(want, got):
            assert torch.equal(a, b)
