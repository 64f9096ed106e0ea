"""Writes tests/golden/config1_golden.json: the oracle's result on the CPU-runnable configuration.

The reference ships no golden vectors, and it cannot be imported here (its imports need axonn,
torch_geometric and ogb).  This fixture is therefore produced by this repository's oracle -- the
reference's operator sequence restated with the same stock torch CPU operators -- in fp64, and serves as
a drift guard: the oracle must keep reproducing it (CPU test) and the device path must match it (GPU test).

    python tests/golden/make_config1_golden.py
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import plexus_oracle as po  # noqa: E402
from plexus_amd.utils import synthetic as S  # noqa: E402


def compute():
    g, x, y, dims = S.config1(device="cpu", seed=0)
    weights = S.glorot_weights(dims, seed=0)
    n = g.shape[0]
    shards = [(g.torch_csr().double(), g.torch_csr(True).double())]
    losses, xf, wf = po.train_epochs(x.double(), [w.double() for w in weights], dims, shards, y, n, 7, epochs=10)
    logits0 = po.OracleNet([w.double() for w in weights], dims).forward(x.double().reshape(-1), shards)
    return {
        "config": "config 1: N=2708, 10556 uniform directed pairs symmetrised + self loops, X Bernoulli(0.013) 2708x1433, "
                  "1433-16-7, Glorot weights, AdamW lr 3e-3, 10 epochs, seed 0",
        "nnz": g.nnz,
        "col_checksum": int(g.col.sum()),
        "val_sum": float(g.val.double().sum()),
        "x_ones": int(x.sum()),
        "label_histogram": torch.bincount(y, minlength=7).tolist(),
        "weight_abs_sum": [float(w.double().abs().sum()) for w in weights],
        "logits_epoch0_abs_sum": float(logits0.abs().sum()),
        "losses_fp64": losses,
        "final_feature_abs_sum": float(xf.abs().sum()),
        "final_weight_abs_sum": [float(w.abs().sum()) for w in wf],
    }


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1_golden.json")
    with open(out, "w") as f:
        json.dump(compute(), f, indent=1)
    print("wrote", out)
