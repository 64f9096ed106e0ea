"""The hot-path entry points are stream-ordered and allocate nothing, so a caller may record them into a HIP graph.

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


@pytest.mark.parametrize("association", ["reference", "auto"])
def test_forward_loss_backward_replay_from_a_hip_graph(association):
    say("HIP graph capture of forward + loss + backward, association=%s" % association)
    n, dims, classes = 3000, [40, 32, 7], 7
    g = S.build_graph(n, "chunglu", 40000, seed=5, device="cpu", gamma=2.1)
    shards = [(to_dev(g, seg_len=64), to_dev(g, True, seg_len=64))]  # split rows: the workspace path is recorded too
    assert shards[0][0].n_long_rows > 0
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
