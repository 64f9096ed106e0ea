"""The C ABI without PyTorch: tests/c_abi/layer_roundtrip is a plain HIP host program that runs one GCN layer
(normalisation, transpose, forward, loss, backward, AdamW) through include/plexus_hip.h and checks every tensor
against the oracle's C routines at the fp32 bar.  It is built beforehand by tests/c_abi/Makefile."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "c_abi", "layer_roundtrip")


@pytest.mark.gpu
def test_layer_roundtrip_program_passes():
    print("[case] C ABI round trip without PyTorch", flush=True)
    assert os.path.exists(BINARY), "build it with `make -C tests/c_abi` (after the library and the oracle)"
    run = subprocess.run([BINARY], capture_output=True, text=True, timeout=110)
    print(run.stdout)
    print(run.stderr)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "all comparisons passed" in run.stdout
    assert run.stdout.count(" ok") >= 13 and "FAILED" not in run.stdout


def test_layer_roundtrip_source_uses_only_the_public_header():
    src = open(os.path.join(HERE, "c_abi", "layer_roundtrip.cpp")).read()
    assert '#include "plexus_hip.h"' in src
    includes = [line.split()[1] for line in src.splitlines() if line.startswith("#include")]
    assert includes == ["<hip/hip_runtime.h>", "<algorithm>", "<cmath>", "<cstdint>", "<cstdio>", "<cstdlib>", "<vector>",
                        '"plexus_hip.h"']


@pytest.mark.gpu
def test_the_reference_side_binding_stub_replaces_torch_sparse_mm():
    """plexus_amd/utils/hip_ops.py is the ctypes stub meant to be copied into the reference tree; it binds the library
    on its own (no other module of this package) and stands in for torch.sparse.mm on a torch CSR tensor."""
    import importlib

    import torch

    from plexus_amd import _lib

    print("[case] reference-side ctypes stub", flush=True)
    os.environ.setdefault("PLEXUS_HIP_LIB", _lib.LIB_PATH)
    stub = importlib.import_module("plexus_amd.utils.hip_ops")
    gen = torch.Generator().manual_seed(0)
    n, d = 3000, 40
    dense = (torch.rand(n, n, generator=gen) < 0.004).float() * torch.rand(n, n, generator=gen)
    a_cpu = dense.to_sparse_csr()
    h = torch.randn(n, d, generator=gen)
    a = a_cpu.to("cuda")
    stub.prepare(a)
    y = stub.sparse_mm(a, h.to("cuda")).cpu()
    ref = torch.sparse.mm(a_cpu, h)
    assert ((y - ref).abs().max() / ref.abs().max()).item() <= 1e-5
