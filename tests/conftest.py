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

    x = torch.as_tensor(x).detach()
    ref = torch.as_tensor(ref).detach()
    # compare where the larger operand already lives (full-size tensors stay on the GPU)
    dev = x.device if x.is_cuda else ref.device
    x = x.to(dev).double()
    ref = ref.to(dev).double()
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


def assert_parity(x, ref32, ref64, tol=FP32_TOL, what=""):
    """fp32 gate with the fp64 oracle as arbiter.

    Passes when x is within `tol` of the fp32 oracle (the reference's own operators on the host) or of the
    fp64 oracle; and, where a long fp32 chain makes the two oracles themselves differ by more than `tol`,
    when x is no further from the fp64 result than the reference's fp32 operators are.
    """
    e32 = rel_err(x, ref32)
    e64 = rel_err(x, ref64)
    ref_gap = rel_err(ref32, ref64)
    print("%s: rel err vs fp32 oracle %.2e, vs fp64 oracle %.2e (fp32 oracle vs fp64 oracle %.2e)" % (what, e32, e64, ref_gap), flush=True)
    assert e32 <= tol or e64 <= tol or e64 <= ref_gap, (
        "%s: rel err vs fp32 oracle %.3e, vs fp64 oracle %.3e, fp32-vs-fp64 oracle gap %.3e" % (what, e32, e64, ref_gap)
    )
