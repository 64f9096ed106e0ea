"""Model and epoch loop of the path: counterpart of examples/train.py:55-112,155-193.

``Net`` stacks GCNConv layers with ReLU after every layer but the last, no bias.  Unlike the reference
(which keeps the layers in a plain list, so the optimizer never sees the weights) the layers are
registered, and the optimizer updates the weights and the input features as the reference's serial
validator does (benchmarking/pyg_serial.py:100-104).
"""
import torch

from . import ops
from .cross_entropy import parallel_cross_entropy
from .gcn_conv import GCNConv
from .optim import AdamW
from .utils.timers import get_timers


class ReluFunction(torch.autograd.Function):
    """The F.relu of examples/train.py:77-78 on the library's kernels, for models that keep it outside the layer:
    forward max(x, 0), backward the upstream gradient where the output is positive."""

    @staticmethod
    def forward(ctx, x):
        y = ops.relu(x.detach())
        ctx.save_for_backward(y)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        (y,) = ctx.saved_tensors
        return ops.relu_bwd(grad_output, y)


def relu(x):
    return ReluFunction.apply(x)


class Net(torch.nn.Module):
    def __init__(self, num_gcn_layers, input_size, hidden_size, output_size, weights=None, fuse_relu=True, dropout=0.0,
                 dropout_seed=0, association="reference"):
        super().__init__()
        self.num_gcn_layers = num_gcn_layers
        self.fuse_relu = fuse_relu
        dims = [input_size] + [hidden_size] * (num_gcn_layers - 1) + [output_size]
        self.layers = torch.nn.ModuleList()
        for i in range(num_gcn_layers):
            last = i == num_gcn_layers - 1
            self.layers.append(
                GCNConv(dims[i], dims[i + 1], i, weight=None if weights is None else weights[i],
                        fuse_relu=fuse_relu and not last, dropout=0.0 if last else dropout, dropout_seed=dropout_seed,
                        association=association)
            )

    def forward(self, x, edge_index_shards):
        for i in range(self.num_gcn_layers):
            x = self.layers[i](x, edge_index_shards)
            if i != self.num_gcn_layers - 1 and not self.fuse_relu:
                x = relu(x)
        return x


def train(model, optimizer, features_local, adj_shards, labels, num_nodes, num_classes):
    """One epoch: examples/train.py:83-112."""
    model.train()
    optimizer.zero_grad()
    output = model(features_local, adj_shards)
    loss = parallel_cross_entropy(output, labels, model.num_gcn_layers, num_nodes, num_classes)
    loss.backward()
    optimizer.step()
    return loss


def make_optimizer(model, features, lr=3e-3, weight_decay=0.0, fused=True, features_bf16=None):
    """AdamW over the weights and the input features (examples/train.py:155-159).

    ``fused`` selects the one-pass kernel of this package; otherwise torch's own optimizer is used.
    With bf16 storage, ``features`` is the fp32 master copy and ``features_bf16`` the tensor the model
    reads (its gradient drives the update and it is refreshed by the same kernel).
    """
    params = list(model.parameters()) + [features]
    if features_bf16 is not None:
        return AdamW(params, lr=lr, weight_decay=weight_decay, shadows=[(features, features_bf16)])
    if fused:
        return AdamW(params, lr=lr, weight_decay=weight_decay)
    return torch.optim.AdamW(params, lr=lr, weight_decay=weight_decay)


def run_epochs(model, optimizer, features, adj_shards, labels, num_nodes, num_classes, num_epochs, log=None):
    """Epoch loop with the reference's per-epoch timer and log line (examples/train.py:164-193)."""
    losses = []
    timers = get_timers()
    for i in range(num_epochs):
        timers.start("epoch " + str(i))
        loss = train(model, optimizer, features, adj_shards, labels, num_nodes, num_classes)
        timers.stop("epoch " + str(i))
        losses.append(float(loss.detach()))
        if log is not None:
            log("Epoch: {:03d}, Train Loss: {:.4f}".format(i, losses[-1]))
    return losses
