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
