"""ctypes binding of libplexus_hip.so -- the C ABI declared in include/plexus_hip.h.

There is no CPU fallback: if the shared library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# PLEXUS_HIP_LIB selects another build of the same ABI (e.g. a tuning variant)
LIB_PATH = os.environ.get("PLEXUS_HIP_LIB") or os.path.join(_HERE, "libplexus_hip.so")

_vp = C.c_void_p
_i64 = C.c_int64
_i32 = C.c_int32
_sz = C.c_size_t
_f32 = C.c_float
_f64 = C.c_double
_u32 = C.c_uint

# name -> (restype, argtypes); mirrors include/plexus_hip.h one to one
SIGNATURES = {
    "plx_version": (C.c_int, []),
    "plx_error_string": (C.c_char_p, [C.c_int]),
    "plx_last_error": (C.c_char_p, []),
    "plx_csr_narrow_i64": (C.c_int, [_i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "plx_csr_transpose_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "plx_csr_transpose_f32": (C.c_int, [_i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "plx_coo_block_to_csr_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "plx_coo_block_to_csr_f32": (C.c_int, [_i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp, C.POINTER(_i64), _vp, _sz, _vp]),
    "plx_invert_permutation_i64": (C.c_int, [_i64, _vp, _vp, _vp]),
    "plx_relabel_edges_i64": (C.c_int, [_i64, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _vp]),
    "plx_csr_to_coo_i64": (C.c_int, [_i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "plx_csr_permute_transposed_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "plx_csr_permute_transposed_f32": (C.c_int, [_i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "plx_gcn_norm_edges_workspace_bytes": (_sz, [_i64, _i64]),
    "plx_gcn_norm_edges_f32": (C.c_int, [_i64, _vp, _vp, _vp, _i64, C.c_int, _vp, _vp, _vp, C.POINTER(_i64), _vp, _sz, _vp]),
    "plx_spmm_segments_host": (C.c_int, [_i64, _vp, _i32, C.POINTER(_i64), C.POINTER(_i64), _vp, _vp, _i64, _vp, _vp, _i64]),
    "plx_spmm_plan_create": (C.c_int, [C.POINTER(_vp), _i64, _i64, _i64, _vp, _vp, _i32, _vp]),
    "plx_spmm_plan_destroy": (C.c_int, [_vp]),
    "plx_spmm_plan_info": (_i64, [_vp, C.c_int]),
    "plx_spmm_plan_tables_host": (C.c_int, [_vp, _vp, _vp, _vp, _vp]),
    "plx_spmm_plan_set_slicing": (C.c_int, [_vp, C.c_int]),
    "plx_spmm_plan_build_hub": (C.c_int, [_vp, _vp]),
    "plx_spmm_plan_build_hub_wide": (C.c_int, [_vp, _vp]),
    "plx_spmm_plan_hub_info": (_i64, [_vp, C.c_int, C.c_int]),
    "plx_spmm_plan_hub_tables_host": (C.c_int, [_vp, C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "plx_spmm_plan_set_hub": (C.c_int, [_vp, C.c_int]),
    "plx_spmm_workspace_bytes": (_sz, [_vp, _i64]),
    "plx_spmm_workspace_bytes_bf16": (_sz, [_vp, _i64]),
    "plx_spmm_csr_f32": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_spmm_csr_rows_f32": (C.c_int, [_vp, _i64, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_spmm_csr_chunk_f32": (C.c_int, [_vp, _i64, _i64, C.c_int, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_spmm_csr_chunk_bf16": (C.c_int, [_vp, _i64, _i64, C.c_int, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_spmm_static_scratch_bytes": (_sz, []),
    "plx_spmm_csr_f32_static": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _vp, _i64, _vp]),
    "plx_spmm_csr_bf16": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_spmm_csr_rows_bf16": (C.c_int, [_vp, _i64, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_gemm_nn_f32": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _u32, _vp]),
    "plx_gemm_f32_split_workspace_bytes": (_sz, [_i64, _i64]),
    "plx_gemm_nn_f32_split": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _u32, _vp, _sz, _vp]),
    "plx_gemm_nt_f32_split": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_gemm_nn_f32_split_bits": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, C.c_uint, _vp, _i64, _vp, _sz, _vp]),
    "plx_gemm_nt_f32_split_bits": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_sign_bits_f32": (C.c_int, [_i64, _i64, _vp, _i64, _vp, _i64, _vp]),
    "plx_gemm_nn_f32_split_dropout": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _u32, _f32, C.c_uint64, C.c_uint64,
                                                _vp, _i64, _vp, _sz, _vp]),
    "plx_gemm_nt_f32_split_scaled": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _f32, _vp, _sz,
                                               _vp]),
    "plx_dropout_f32": (C.c_int, [_i64, _i64, _vp, _i64, _f32, C.c_uint64, C.c_uint64, _vp]),
    "plx_gemm_nt_f32": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "plx_gemm_tn_f32_split_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "plx_gemm_tn_f32_split": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _f32, _vp, _sz, _vp]),
    "plx_gemm_tn_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "plx_gemm_tn_f32": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _sz, _vp]),
    "plx_copy_rows": (C.c_int, [_i64, _i64, _vp, _i64, _vp, _i64, _vp]),
    "plx_relu_f32": (C.c_int, [_i64, _i64, _vp, _i64, _vp, _i64, _vp]),
    "plx_relu_bwd_f32": (C.c_int, [_i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "plx_softmax_xent_workspace_bytes": (_sz, [_i64, _i64]),
    "plx_softmax_xent_f32": (C.c_int, [_i64, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _f32, _vp, _vp, _i64, _vp, _sz, _vp]),
    "plx_scale_by_device_scalar_f32": (C.c_int, [_i64, _vp, _vp, _vp, _vp]),
    "plx_scale_by_device_scalar_bf16": (C.c_int, [_i64, _vp, _vp, _vp, _vp]),
    "plx_gcn_norm_csr_f32": (C.c_int, [_i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "plx_adamw_f32": (C.c_int, [_i64, _vp, _vp, _vp, _vp, _f64, _f64, _f64, _f64, _f64, _i64, _vp]),
    "plx_adamw_f32_grad_bf16": (C.c_int, [_i64, _vp, _vp, _vp, _vp, _f64, _f64, _f64, _f64, _f64, _i64, _vp, _vp]),
    "plx_gemm_nt_bf16": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _f32, _u32, _f32,
                                   C.c_uint64, C.c_uint64, _vp]),
    "plx_gemm_tn_bf16_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "plx_gemm_tn_bf16": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _f32, _vp, _sz, _vp]),
    "plx_gemm_nt_bf16_bits": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _f32, _u32,
                                        _f32, C.c_uint64, C.c_uint64, _vp]),
    "plx_gemm_tn_bf16_bits": (C.c_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _f32, _vp, _sz, _vp]),
    "plx_cast_f32_bf16": (C.c_int, [_i64, _i64, _vp, _i64, _vp, _i64, C.c_int, _vp]),
    "plx_softmax_xent_bf16": (C.c_int, [_i64, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _f32, _vp, _vp, _i64, _vp, _sz, _vp]),
}

# include/plexus_hip_diag.h: measurement probes, not part of the path
DIAG_SIGNATURES = {
    "plx_diag_random_gather_f32": (C.c_int, [_vp, _i64, _i64, _i64, _i64, C.POINTER(_i64), _vp, _vp]),
    "plx_diag_spmm_parts_f32": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _vp, _i64, _vp, C.c_size_t, C.c_int, _vp]),
}

PLX_GEMM_RELU = 1
PLX_GEMM_DROPOUT = 2
# plx_status of include/plexus_hip.h
PLX_OK, PLX_ERR_INVALID, PLX_ERR_HIP, PLX_ERR_WORKSPACE, PLX_ERR_UNSUPPORTED, PLX_ERR_NOMEM = 0, -1, -2, -3, -4, -5

_lib = None


class PlexusHipError(RuntimeError):
    """A libplexus_hip entry point returned a negative status."""


def load():
    """Load the shared library once.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise PlexusHipError(
                f"{LIB_PATH} is missing: build it with `make -C plexus_amd/csrc` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no CPU fallback"
            )
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in list(SIGNATURES.items()) + list(DIAG_SIGNATURES.items()):
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        lib = load()
        raise PlexusHipError(
            f"{what}: {lib.plx_error_string(status).decode()} ({status}): {lib.plx_last_error().decode()}"
        )
