import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box with -m gpu)")


def rel_err(x, ref):
    """max|x - ref| / max|ref| -- the parity measure of every fp32 / bf16 comparison in this suite."""
    import torch

    x = torch.as_tensor(x).detach().double().cpu()
    ref = torch.as_tensor(ref).detach().double().cpu()
    denom = ref.abs().max().item()
    if denom == 0.0:
        return (x - ref).abs().max().item()
    return (x - ref).abs().max().item() / denom


FP32_TOL = 1e-5  # max relative error for fp32 outputs
BF16_TOL = 2e-2  # bf16 storage with fp32 accumulation


@pytest.fixture(scope="session")
def lib():
    from plexus_amd import _lib

    return _lib.load()
