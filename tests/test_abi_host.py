"""CPU-only checks of the boundary: the shared library loads, exports what the header declares,
reports errors without a GPU, and its host-side row analysis is correct."""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

from plexus_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols(name="plexus_hip.h"):
    text = open(os.path.join(ROOT, "include", name)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(plx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    syms = header_symbols()
    assert len(syms) >= 18
    for s in syms:
        assert hasattr(lib, s), "libplexus_hip.so does not export %s" % s
    # and the Python binding table covers exactly the header
    assert sorted(_lib.SIGNATURES) == syms
    # the measurement probes live in their own header
    diag = header_symbols("plexus_hip_diag.h")
    assert sorted(_lib.DIAG_SIGNATURES) == diag and not set(diag) & set(syms)
    for s in diag:
        assert hasattr(lib, s), "libplexus_hip.so does not export %s" % s


def header_prototypes():
    """name -> (return type, [parameter types]) as written in the header, comments and names stripped."""
    text = open(os.path.join(ROOT, "include", "plexus_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = {}
    for ret, name, params in re.findall(r"^\s*([a-z_0-9 ]+?\*?)\s*\b(plx_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text, flags=re.M | re.S):
        types = []
        for prm in [x.strip() for x in params.replace("\n", " ").split(",")]:
            if prm in ("void", ""):
                continue
            types.append("ptr" if "*" in prm else re.sub(r"\s+\w+$", "", prm.replace("const ", "")).strip())
        protos[name] = (ret.strip(), types)
    return protos


def test_binding_table_matches_the_header_types():
    """Every ctypes signature has the arity and the scalar types of its C prototype (a float/double or
    int32/int64 slip corrupts arguments silently)."""
    scalar = {"int64_t": C.c_int64, "int32_t": C.c_int32, "int": C.c_int, "unsigned": C.c_uint, "float": C.c_float,
              "double": C.c_double, "size_t": C.c_size_t, "uint64_t": C.c_uint64}
    rets = {"int": C.c_int, "size_t": C.c_size_t, "int64_t": C.c_int64, "const char *": C.c_char_p, "const char*": C.c_char_p}
    protos = header_prototypes()
    assert sorted(protos) == sorted(_lib.SIGNATURES)
    for name, (ret, types) in protos.items():
        res, args = _lib.SIGNATURES[name]
        assert rets[ret] is res, name
        assert len(args) == len(types), "%s: %d parameters in the header, %d in the binding" % (name, len(types), len(args))
        for i, (t, a) in enumerate(zip(types, args)):
            if t == "ptr":
                assert a is C.c_void_p or issubclass(a, C._Pointer) or a is C.c_char_p, "%s arg %d" % (name, i)
            else:
                assert scalar[t] is a, "%s arg %d: header %s, binding %s" % (name, i, t, a)


def test_version_and_error_strings(lib):
    assert lib.plx_version() >= 100
    assert lib.plx_error_string(0) == b"ok"
    assert b"workspace" in lib.plx_error_string(-3)
    assert lib.plx_error_string(-99) == b"unknown status"


def test_argument_errors_are_reported_not_thrown(lib):
    # negative sizes / NULL pointers are rejected before any device work
    rc = lib.plx_gemm_nn_f32(-1, 4, 4, None, 4, None, 4, None, 4, 0, None)
    assert rc == -1 and b"negative" in lib.plx_last_error()
    rc = lib.plx_spmm_csr_f32(None, None, None, 4, 4, None, 4, None, 0, None)
    assert rc == -1 and b"plan is NULL" in lib.plx_last_error()
    rc = lib.plx_softmax_xent_f32(4, 2000, None, 2000, None, 4, 2000, 0, 1.0, None, None, 2000, None, 0, None)
    assert rc == -1 and b"classes" in lib.plx_last_error()
    with pytest.raises(_lib.PlexusHipError):
        _lib.check(rc, "plx_softmax_xent_f32")


def segments(rowptr, seg_len):
    lib = _lib.load()
    rp = np.ascontiguousarray(rowptr, dtype=np.int32)
    m = rp.size - 1
    nl, ns = C.c_int64(), C.c_int64()
    rc = lib.plx_spmm_segments_host(m, rp.ctypes.data, seg_len, C.byref(nl), C.byref(ns), None, None, 0, None, None, 0)
    assert rc == 0
    lr = np.zeros(nl.value, np.int32)
    sf = np.zeros(nl.value + 1, np.int32)
    sb = np.zeros(ns.value, np.int32)
    se = np.zeros(ns.value, np.int32)
    rc = lib.plx_spmm_segments_host(m, rp.ctypes.data, seg_len, C.byref(nl), C.byref(ns), lr.ctypes.data, sf.ctypes.data,
                                    nl.value, sb.ctypes.data, se.ctypes.data, ns.value)
    assert rc == 0
    return lr, sf, sb, se


def test_row_segments_cover_long_rows_exactly():
    rng = np.random.default_rng(0)
    lens = rng.integers(0, 40, size=500)
    lens[[3, 77, 401]] = [1000, 64 * 9 + 1, 65]
    lens[10] = 64
    rowptr = np.concatenate([[0], np.cumsum(lens)])
    lr, sf, sb, se = segments(rowptr, 64)
    assert list(lr) == [3, 77, 401]  # rows of exactly seg_len stay whole
    assert sf[0] == 0 and sf[-1] == sb.size
    for q, r in enumerate(lr):
        b, e = sb[sf[q]:sf[q + 1]], se[sf[q]:sf[q + 1]]
        assert b[0] == rowptr[r] and e[-1] == rowptr[r + 1]
        assert (b[1:] == e[:-1]).all()  # contiguous, ordered
        ln = e - b
        assert ln.max() <= 64 and ln.max() - ln.min() <= 1  # balanced
        assert ln.size == -(-lens[r] // 64)
    # no long rows -> nothing to do
    lr, sf, sb, se = segments(np.arange(0, 50, 5), 64)
    assert lr.size == 0 and sb.size == 0 and list(sf) == [0]


def test_row_segments_reject_decreasing_rowptr(lib):
    rp = np.array([0, 5, 3], dtype=np.int32)
    nl, ns = C.c_int64(), C.c_int64()
    rc = lib.plx_spmm_segments_host(2, rp.ctypes.data, 4, C.byref(nl), C.byref(ns), None, None, 0, None, None, 0)
    assert rc == -1 and b"decreases" in lib.plx_last_error()


def test_workspace_queries_without_gpu(lib):
    assert lib.plx_spmm_workspace_bytes(None, 128) == 0
    assert lib.plx_gemm_tn_workspace_bytes(0, 4, 4) == 0
    small = lib.plx_gemm_tn_workspace_bytes(100, 16, 16)
    big = lib.plx_gemm_tn_workspace_bytes(2449029, 128, 128)
    assert small == 0 and big > 0 and big % (128 * 128 * 4) == 0
    assert lib.plx_softmax_xent_workspace_bytes(10, 10) > 0


def test_init_keeps_reference_keywords_and_rejects_grids():
    import plexus_amd
    from plexus_amd import plexus as plx

    plexus_amd.init(G_intra_r=1, G_intra_c=1, G_intra_d=1, gpus_per_node=None, enable_internal_timers=False,
                    block_aggregation=True, overlap_aggregation=True, tune_gemms=True)
    assert plx.block_agg and plx.overlap_agg and plx.tune_gemm
    with pytest.raises(AssertionError):  # overlap needs blocking, as in the reference
        plexus_amd.init(overlap_aggregation=True)
    with pytest.raises(ValueError):
        plexus_amd.init(G_intra_r=2)
    plexus_amd.init()
    assert not plx.block_agg


def test_host_helpers():
    from plexus_amd.gcn_conv import GCNConv, chunk_bounds
    from plexus_amd.utils.general import pad_dimension, set_seed
    from plexus_amd.utils.matmul_tuning import _is_transposed_view

    assert pad_dimension(10, 4) == 12 and pad_dimension(7, 2, 3) == 12 and pad_dimension(8, 1) == 8
    assert chunk_bounds(2449029) == [(0, 816343), (816343, 1632686), (1632686, 2449029)]
    a = torch.zeros(5, 3)
    assert _is_transposed_view(a.t()) and not _is_transposed_view(a)
    set_seed(0)
    l0 = GCNConv(100, 16, 0, device="cpu")
    set_seed(0)
    l1 = GCNConv(100, 16, 0, device="cpu")
    assert l0.weight.shape == (1600,) and torch.equal(l0.weight, l1.weight)
    assert l0.weight.abs().max() <= 0.25  # bound 1 / sqrt(out_channels)
    assert l0.gather_features and not GCNConv(4, 4, 1, device="cpu").gather_features


def test_product_path_refuses_cpu_tensors():
    from plexus_amd import ops

    with pytest.raises(_lib.PlexusHipError):
        ops.gemm_nn(torch.zeros(4, 4), torch.zeros(4, 4))
