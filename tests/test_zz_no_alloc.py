"""The SpMM entry point that allocates nothing (plx_spmm_csr_f32_static): partial sums of the split rows live in a
static device array instead of a caller's workspace.  Checked bit for bit against plx_spmm_csr_f32 through the C ABI,
on two calls in a row (the second smaller, so the array still holds the first call's partial rows), and against the
fp64 oracle.  Collected last on purpose: a failure here must not hide the tests of the path itself."""
import pytest
import torch

from conftest import FP32_TOL, rel_err
from oracle import oracle_c
from plexus_amd import _lib, ops
from plexus_amd.utils import synthetic as S

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _both(lib, g, d, seg_len, seed):
    a = ops.CsrMatrix(g.rowptr.to(DEV), g.col.to(DEV), g.val.to(DEV), g.shape, seg_len)
    assert a.n_long_rows > 0 and a.n_segments >= 2 * a.n_long_rows
    h_host = torch.randn(g.shape[1], d, generator=torch.Generator().manual_seed(seed))
    h = h_host.to(DEV)
    m = g.shape[0]
    y_ref = ops.spmm(a, h)  # plx_spmm_csr_f32 with a caller's workspace
    y = torch.full((m, d), float("nan"), device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.plx_spmm_csr_f32_static(a._plan, a.val.data_ptr(), h.data_ptr(), d, d, y.data_ptr(), d, stream)
    _lib.check(rc, "plx_spmm_csr_f32_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(y, y_ref)
    ref64 = oracle_c.csr_spmm(g.rowptr.numpy(), g.col.numpy(), g.val.numpy(), h_host.numpy())
    assert rel_err(y.cpu(), ref64) <= FP32_TOL
    return a


def test_static_scratch_spmm_two_calls_second_smaller():
    lib = _lib.load()
    assert lib.plx_spmm_static_scratch_bytes() == 32 << 20
    print("[case] static-scratch spmm: 3000 nodes D=128 seg_len=64, then 1200 nodes D=40 seg_len=16", flush=True)
    big = S.build_graph(3000, "chunglu", 40000, seed=1, device="cpu", gamma=2.1)
    small = S.build_graph(1200, "chunglu", 9000, seed=2, device="cpu", gamma=2.1)
    _both(lib, big, 128, 64, seed=3)
    _both(lib, small, 40, 16, seed=4)
    # and once more on the larger one: the array now holds the smaller call's rows
    _both(lib, big, 602, 256, seed=5)


def test_static_scratch_spmm_refuses_what_does_not_fit():
    lib = _lib.load()
    print("[case] static-scratch spmm: plan whose partial rows exceed the array", flush=True)
    g = S.build_graph(3000, "chunglu", 40000, seed=1, device="cpu", gamma=2.1)
    a = ops.CsrMatrix(g.rowptr.to(DEV), g.col.to(DEV), g.val.to(DEV), g.shape, 4)
    d = 2048
    assert a.n_segments * d * 4 > (32 << 20)
    h = torch.zeros(3000, d, device=DEV)
    y = torch.zeros(3000, d, device=DEV)
    rc = lib.plx_spmm_csr_f32_static(a._plan, a.val.data_ptr(), h.data_ptr(), d, d, y.data_ptr(), d,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.PLX_ERR_WORKSPACE
    assert b"static" in lib.plx_last_error()
    with pytest.raises(_lib.PlexusHipError, match="workspace"):
        _lib.check(rc, "plx_spmm_csr_f32_static")


def test_static_scratch_spmm_on_a_plan_with_a_hub_pass():
    """The static entry point never takes the hub pass: bit for bit the product with the pass switched off, and within
    fp32 rounding of the product that takes it."""
    lib = _lib.load()
    print("[case] static-scratch spmm on a plan with hub tables", flush=True)
    g = S.build_graph(3000, "chunglu", 40000, seed=7, device="cpu", gamma=2.1)
    a = ops.CsrMatrix(g.rowptr.to(DEV), g.col.to(DEV), g.val.to(DEV), g.shape, 16)
    a.build_hub()
    assert a.n_hub_rows > 0
    d = 128
    h = torch.randn(3000, d, generator=torch.Generator().manual_seed(8)).to(DEV)
    y_hub = ops.spmm(a, h)
    a.set_hub(-1)
    y_plain = ops.spmm(a, h)
    a.set_hub(0)
    assert not torch.equal(y_hub, y_plain)
    y = torch.full((3000, d), float("nan"), device=DEV)
    _lib.check(lib.plx_spmm_csr_f32_static(a._plan, a.val.data_ptr(), h.data_ptr(), d, d, y.data_ptr(), d,
                                           torch.cuda.current_stream().cuda_stream), "plx_spmm_csr_f32_static")
    assert torch.equal(y, y_plain)
    assert rel_err(y.cpu(), y_hub.cpu()) <= 2e-6
