"""The binding a maintainer of the reference adds to swap its sparse product for libplexus_hip's.

Self-contained on purpose (ctypes and torch only, nothing else of this package): copied to
``plexus/utils/hip_ops.py`` in the reference tree, ``prepare(a)`` is called once per CSR shard at the end of
``DataLoader.__split_adj`` (plexus/utils/dataloader.py:343-375) and ``sparse_mm(a, h)`` replaces
``torch.sparse.mm(a, h)`` at plexus/gcn_conv.py:98, :188 and :265.  ``PLEXUS_HIP_LIB`` names the library when it
is not on the loader's search path.
"""
import ctypes
import os

import torch

_lib = ctypes.CDLL(os.environ.get("PLEXUS_HIP_LIB", "libplexus_hip.so"))
_lib.plx_last_error.restype = ctypes.c_char_p
_lib.plx_spmm_plan_create.argtypes = [ctypes.POINTER(ctypes.c_void_p)] + [ctypes.c_int64] * 3 + \
    [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p]
_lib.plx_spmm_workspace_bytes.restype = ctypes.c_size_t
_lib.plx_spmm_workspace_bytes.argtypes = [ctypes.c_void_p, ctypes.c_int64]
_lib.plx_spmm_csr_f32.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int64] * 2 + [ctypes.c_void_p, ctypes.c_int64,
                                  ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]


def prepare(a):
    """Once per CSR shard: int32 indices and the row plan, kept on the tensor."""
    rp = a.crow_indices().to(torch.int32)
    ci = a.col_indices().to(torch.int32)
    plan = ctypes.c_void_p()
    rc = _lib.plx_spmm_plan_create(ctypes.byref(plan), a.shape[0], a.shape[1], ci.numel(), rp.data_ptr(),
                                   ci.data_ptr(), 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.plx_last_error()
    a._hip = (plan, rp, ci, a.values().contiguous())  # the int32 arrays must live as long as the plan


def sparse_mm(a, h):
    """torch.sparse.mm(a, h) for a prepared CSR tensor ``a`` and a row-major fp32 ``h`` on the same GPU."""
    plan, rp, ci, val = a._hip
    y = torch.empty(a.shape[0], h.shape[1], device=h.device)
    n = _lib.plx_spmm_workspace_bytes(plan, h.shape[1])
    ws = torch.empty(max(n, 1), dtype=torch.uint8, device=h.device)
    rc = _lib.plx_spmm_csr_f32(plan, val.data_ptr(), h.data_ptr(), h.stride(0), h.shape[1], y.data_ptr(),
                               y.stride(0), ws.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.plx_last_error()
    return y
