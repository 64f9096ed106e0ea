"""The benchmark networks end to end on the GPU against the CPU oracle: the 100-128-128-47 fp32 network of the
2.45 M-node power-law configuration (forward, loss, backward; a tenth of the size against the fp32 and fp64 oracles,
full size against the same), and ten AdamW epochs of that network and of the bf16 / dropout network (loss per epoch).

fp32 bar: 1e-5 (max|x - ref| / max|ref| per tensor, |loss - ref| / |ref| per epoch), fp64 oracle as arbiter;
bf16 storage: 2e-2.
"""
import pytest
import torch

from conftest import BF16_TOL, FP32_TOL, assert_parity, rel_err
from oracle import plexus_oracle as po
from plexus_amd import ops
from plexus_amd.utils import synthetic as S

pytestmark = pytest.mark.gpu
DEV = "cuda"
DIMS3 = [100, 128, 128, 47]


def say(msg):
    print("[case] " + msg, flush=True)


def host_csr_pair(g, dtype=torch.float32):
    a = torch.sparse_csr_tensor(g.rowptr.cpu(), g.col.cpu(), g.val.cpu().to(dtype), size=g.shape)
    at = torch.sparse_csr_tensor(g.rowptr_t.cpu(), g.col_t.cpu(), g.val_t.cpu().to(dtype), size=(g.shape[1], g.shape[0]))
    return a, at


def device_csr_pair(g):
    return (ops.CsrMatrix(g.rowptr, g.col, g.val, g.shape), ops.CsrMatrix(g.rowptr_t, g.col_t, g.val_t, (g.shape[1], g.shape[0])))


def network_forward_loss_backward(scale, max_flips, g=None, DIMS3=DIMS3):
    """One forward + loss + backward of a three-layer fp32 network, every tensor of it against the oracle."""
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.gcn_conv import GCNConv

    if g is None:
        g = S.config3_graph(DEV, seed=0, scale=scale)
    n = g.shape[0]
    assert g.shape[0] == g.shape[1]
    print(g.degree_stats(), flush=True)
    x = S.normal_features(n, DIMS3[0], DEV, seed=1)
    y = S.uniform_labels(n, DIMS3[-1], DEV, seed=2)
    ws = S.glorot_weights(DIMS3, seed=0)
    shards = [device_csr_pair(g)]

    layers = [GCNConv(DIMS3[i], DIMS3[i + 1], i, weight=ws[i], fuse_relu=(i < 2)) for i in range(3)]
    xd = x.reshape(-1).clone().requires_grad_()  # flat, as layer 0 receives it
    h = xd
    acts = []
    for layer in layers:
        h = layer(h, shards)
        acts.append(h)
    loss = parallel_cross_entropy(h, y, 3, n, DIMS3[-1])
    loss.backward()
    torch.cuda.synchronize()

    x_cpu, y_cpu = x.cpu(), y.cpu()
    pair32, pair64 = host_csr_pair(g), host_csr_pair(g, torch.float64)
    net = po.OracleNet(ws, DIMS3)
    logits_ref = net.forward(x_cpu.reshape(-1), [pair32])
    net64 = po.OracleNet([w.double() for w in ws], DIMS3)
    logits64 = net64.forward(x_cpu.double().reshape(-1), [pair64])
    loss_ref, sm, oh = po.cross_entropy_forward(logits_ref, y_cpu, n, DIMS3[-1])
    loss64, sm64, oh64 = po.cross_entropy_forward(logits64, y_cpu, n, DIMS3[-1])
    print("loss gpu %.7f, oracle fp32 %.7f, fp64 %.7f" % (loss.item(), loss_ref.item(), loss64.item()), flush=True)
    assert abs(loss.item() - loss64.item()) <= FP32_TOL * abs(loss64.item())
    assert abs(loss.item() - loss_ref.item()) <= FP32_TOL * abs(loss_ref.item())
    assert_parity(acts[2], logits_ref, logits64, what="logits")

    # hidden activations, and the ReLU masks the backward pass is pinned to: a pre-activation within rounding of zero
    # may take either sign in two fp32 summation orders
    masks = []
    for i in range(2):
        mask = (acts[i] > 0).cpu()
        flips = int((mask != (net64._saved[i][3] > 0)).sum())
        print("layer %d: %d of %d ReLU mask elements differ from the fp64 oracle" % (i, flips, mask.numel()), flush=True)
        assert flips <= max_flips
        assert_parity(acts[i], torch.relu(net._saved[i][3]), torch.relu(net64._saved[i][3]), what="hidden %d" % i)
        masks.append(mask)
    masks.append(None)
    gl = po.cross_entropy_backward(sm, oh.float(), n)
    gl64 = po.cross_entropy_backward(sm64, oh64.double(), n)
    gx_ref, gws_ref = net.backward(gl, masks)
    gx64, gws64 = net64.backward(gl64, masks)
    assert xd.grad.shape == (n * DIMS3[0],)
    assert_parity(xd.grad, gx_ref, gx64, what="grad_x")
    for i, layer in enumerate(layers):
        assert layer.weight.grad.shape == (DIMS3[i] * DIMS3[i + 1],)
        assert_parity(layer.weight.grad, gws_ref[i], gws64[i], what="grad_w[%d]" % i)


def test_config3_network_forward_loss_backward_at_a_tenth():
    say("config 3 network 100-128-128-47 fp32, 1/10 scale: logits, loss, hidden activations, grad_x, grad_w")
    network_forward_loss_backward(0.1, max_flips=8)


def test_config3_network_forward_loss_backward_full_size():
    say("config 3 network 100-128-128-47 fp32, full size (2.45 M nodes): logits, loss, hidden activations, grad_x, grad_w")
    network_forward_loss_backward(1.0, max_flips=80)


def test_config4_rank_block_network_full_size():
    """One rank's block of a 2 x 2 x 2 grid at its real shape (rows and columns [0, N/2) of a doubly permuted R-MAT graph with
    N = 8,388,608: 4,194,304 x 4,194,304, about 64 M entries, not symmetric), local widths 64 -> 64 -> 64 -> 24: forward,
    loss and backward of the three layers against the oracle in fp32 and fp64."""
    say("config 4 block network 64-64-64-24 fp32, full size")
    g = S.config4_block(DEV, seed=0, scale=1.0)
    assert not torch.equal(g.rowptr, g.rowptr_t)
    network_forward_loss_backward(1.0, max_flips=80, g=g, DIMS3=[64, 64, 64, 24])


def test_config5_network_full_size_bf16_dropout():
    """The bf16-storage 256-256-256-47 network with dropout 0.5 at full size (2.45 M nodes): logits, loss, grad_x and the
    three grad_w against the bf16-storage oracle, which regenerates the dropout masks from the same seed and offsets."""
    say("config 5 network 256-256-256-47 bf16 + dropout, full size")
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.train import Net

    dims, seed = [256, 256, 256, 47], 11
    g = S.config3_graph(DEV, seed=0, scale=1.0)
    n = g.shape[0]
    x = S.normal_features(n, dims[0], DEV, seed=1)
    y = S.uniform_labels(n, dims[-1], DEV, seed=2)
    ws = S.glorot_weights(dims, seed=0)
    model = Net(3, dims[0], dims[1], dims[-1], weights=ws, fuse_relu=True, dropout=0.5, dropout_seed=seed)
    model.train()
    offsets = [layer.next_dropout_offset() for layer in model.layers]
    xd = x.to(torch.bfloat16).requires_grad_()
    logits = model(xd, [device_csr_pair(g)])
    loss = parallel_cross_entropy(logits, y, 3, n, dims[-1])
    loss.backward()
    torch.cuda.synchronize()

    net = po.OracleNetBf16(ws, dims, dropout_p=0.5, seed=seed)
    ref_logits = net.forward(x.cpu(), [host_csr_pair(g)], offsets)
    ref_loss, sm, oh = po.cross_entropy_forward(ref_logits, y.cpu(), n, dims[-1])
    gx_ref, gws_ref = net.backward(po.cross_entropy_backward(sm, oh.float(), n))
    errs = {"logits": rel_err(logits.float(), ref_logits), "loss": abs(loss.item() - ref_loss.item()) / abs(ref_loss.item()),
            "grad_x": rel_err(xd.grad.float(), gx_ref.reshape(n, dims[0]))}
    for i, (layer, gw) in enumerate(zip(model.layers, gws_ref)):
        errs["grad_w[%d]" % i] = rel_err(layer.weight.grad, gw)
    print("loss gpu %.6f oracle %.6f; rel errors %s" % (loss.item(), ref_loss.item(), {k: "%.2e" % v for k, v in errs.items()}), flush=True)
    assert all(v <= BF16_TOL for v in errs.values()), errs


def test_config3_ten_epoch_loss_curve():
    """Ten AdamW epochs (weights and features trained) of the fp32 network at 1/20 of the size: the loss of every
    epoch against the oracle's loop in fp32 and fp64."""
    say("config 3 network, 1/20 scale, 10 epochs")
    from plexus_amd.train import Net, make_optimizer, run_epochs

    g = S.config3_graph(DEV, seed=0, scale=0.05)
    n = g.shape[0]
    x = S.normal_features(n, DIMS3[0], DEV, seed=1)
    y = S.uniform_labels(n, DIMS3[-1], DEV, seed=2)
    ws = S.glorot_weights(DIMS3, seed=0)
    model = Net(3, DIMS3[0], DIMS3[1], DIMS3[-1], weights=ws, fuse_relu=True)
    feats = x.reshape(-1).clone().requires_grad_()
    # the ReLU masks of every epoch, for the comparison of the trained tensors below
    masks = [[], []]
    for i in range(2):
        model.layers[i].register_forward_hook(lambda mod, args, out, i=i: masks[i].append(out.detach() > 0))
    losses = run_epochs(model, make_optimizer(model, feats), feats, [device_csr_pair(g)], y, n, DIMS3[-1], 10)

    pair32, pair64 = host_csr_pair(g), host_csr_pair(g, torch.float64)
    w64_0 = [w.double() for w in ws]
    ref32, _, _ = po.train_epochs(x.cpu(), ws, DIMS3, [pair32], y.cpu(), n, DIMS3[-1], epochs=10)
    ref64, _, _ = po.train_epochs(x.cpu().double(), w64_0, DIMS3, [pair64], y.cpu(), n, DIMS3[-1], epochs=10)
    print("gpu   ", ["%.6f" % v for v in losses], flush=True)
    print("fp32  ", ["%.6f" % v for v in ref32], flush=True)
    print("fp64  ", ["%.6f" % v for v in ref64], flush=True)
    for e, (l, r32, r64) in enumerate(zip(losses, ref32, ref64)):
        assert abs(l - r64) <= FP32_TOL * abs(r64) or abs(l - r32) <= FP32_TOL * abs(r32), "epoch %d" % e
    assert losses[-1] < losses[0]
    # The trained tensors.  A hidden unit whose pre-activation is within rounding of zero takes either side of the ReLU in
    # two fp32 summation orders, and through a hub vertex one such unit reaches most features; so the oracle's backward
    # passes are given the masks the GPU run produced (a handful of elements differ from the oracle's own), and then
    # the trained features and weights must agree like any other fp32 tensor.
    picked = lambda e: [masks[0][e].cpu(), masks[1][e].cpu(), None]
    m32, x32, w32 = po.train_epochs(x.cpu(), ws, DIMS3, [pair32], y.cpu(), n, DIMS3[-1], epochs=10, masks_of_epoch=picked)
    m64, x64, w64 = po.train_epochs(x.cpu().double(), w64_0, DIMS3, [pair64], y.cpu(), n, DIMS3[-1], epochs=10, masks_of_epoch=picked)
    assert max(abs(u - v) for u, v in zip(m64, ref64)) <= 1e-6  # pinning the masks barely moves the oracle's losses (gate: 4e-5)
    assert_parity(feats, x32, x64, what="trained features")
    # Weights: an element of GRAD_W is a sum over all vertices that cancels to ~1e-7 for some elements, the size of Adam's
    # eps (1e-8) and of the rounding noise of any fp32 summation order (seen: grad_w agrees to 2.6e-6 of its largest
    # element, the reference's own fp32 operators to 1.3e-6); the update lr * m / (sqrt(v) + eps) of such an element
    # turns that noise into a few 1e-6 of absolute difference per step.  A dozen elements per matrix end up to 8e-6 away
    # after ten steps (4e-5 of the largest weight; the same with torch.optim.AdamW in place of the fused kernel), every other
    # one within 1e-6: the bar for the trained weights is 1e-4 of the largest element.
    for i, layer in enumerate(model.layers):
        assert_parity(layer.weight, w32[i], w64[i], tol=1e-4, what="trained weight %d" % i)
        d = (layer.weight.detach().cpu().double() - w64[i]).abs()
        assert (d > 2e-6).sum().item() <= 64, "trained weight %d: %d elements more than 2e-6 away" % (i, int((d > 2e-6).sum()))


def test_config5_ten_epoch_loss_curve_bf16_dropout():
    """Ten AdamW epochs of the bf16-storage 256-256-256-47 network with dropout 0.5 at 1/100 of the size: fp32 master
    features and weights, bf16 activations and gradients; the oracle regenerates every epoch's dropout masks from the
    same seed and offsets."""
    say("config 5 network, 1/100 scale, bf16 storage, dropout 0.5, 10 epochs")
    from plexus_amd.train import Net, make_optimizer, run_epochs

    dims, seed = [256, 256, 256, 47], 7
    g = S.config3_graph(DEV, seed=1, scale=0.01)
    n = g.shape[0]
    x = S.normal_features(n, dims[0], DEV, seed=1)
    y = S.uniform_labels(n, dims[-1], DEV, seed=2)
    ws = S.glorot_weights(dims, seed=2)
    model = Net(3, dims[0], dims[1], dims[-1], weights=ws, fuse_relu=True, dropout=0.5, dropout_seed=seed)
    master = x.reshape(-1).clone()
    shadow = master.to(torch.bfloat16).requires_grad_()
    offsets_seen = []
    opt = make_optimizer(model, master, features_bf16=shadow)

    def log(_):
        offsets_seen.append([layer.next_dropout_offset() for layer in model.layers])

    log(None)
    losses = run_epochs(model, opt, shadow, [device_csr_pair(g)], y, n, dims[-1], 10, log=log)
    offs = lambda e: offsets_seen[e]  # what each layer used in epoch e (read before the epoch ran)
    assert offsets_seen[1][0] != offsets_seen[0][0]
    ref, x_ref, w_ref = po.train_epochs_bf16(x.cpu(), ws, dims, [host_csr_pair(g)], y.cpu(), n, dims[-1], epochs=10, dropout_p=0.5,
                                             seed=seed, offsets_of_epoch=offs)
    print("gpu   ", ["%.5f" % v for v in losses], flush=True)
    print("oracle", ["%.5f" % v for v in ref], flush=True)
    for e, (l, r) in enumerate(zip(losses, ref)):
        assert abs(l - r) <= BF16_TOL * abs(r), "epoch %d" % e
    assert losses[-1] < losses[0]
    assert rel_err(master, x_ref) <= BF16_TOL
    assert torch.equal(shadow.detach(), master.to(torch.bfloat16))  # the update refreshed the copy the model reads
    # Weights: every Adam step moves an element by about +-lr whatever the size of its gradient, so an element whose
    # gradient is within the bf16 noise of zero walks differently in the two runs.  Compared are the movements: those of
    # the two runs must be close on the whole (relative l2 distance), and few elements may be a whole step apart.
    for i, (layer, w, w0) in enumerate(zip(model.layers, w_ref, ws)):
        mine = layer.weight.detach().cpu().double() - w0.double().reshape(-1)
        ref_move = w.double().reshape(-1) - w0.double().reshape(-1)
        dist = ((mine - ref_move).norm() / ref_move.norm()).item()
        far = ((mine - ref_move).abs() > 3e-3).double().mean().item()
        print("weight %d: movement l2 distance %.3f of the oracle's movement, %.3f %% of the elements more than one step lr apart, "
              "max %.1f steps" % (i, dist, 100 * far, (mine - ref_move).abs().max().item() / 3e-3), flush=True)
        assert dist <= 0.15 and far <= 0.04
