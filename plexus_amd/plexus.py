"""Configuration entry point; same keyword arguments as the reference's plexus/plexus.py:5-48.

The reference hands the grid sizes to AxoNN to create process groups.  This build runs on one GPU:
a grid other than 1 x 1 x 1 is rejected.  The three module globals the operator layer reads
(``block_agg``, ``overlap_agg``, ``tune_gemm``; plexus/plexus.py:43-48) are kept.
"""
from typing import Optional

from .utils import timers as _timers

block_agg = False
overlap_agg = False
tune_gemm = False
_initialized = False


def init(G_intra_r: int = 1, G_intra_c: int = 1, G_intra_d: int = 1, gpus_per_node: Optional[int] = None,
         enable_internal_timers: bool = False, block_aggregation: bool = False, overlap_aggregation: bool = False,
         tune_gemms: bool = False) -> None:
    """Initialise the (one-GPU) runtime.

    Arguments keep the reference's meaning.  ``G_intra_r/c/d`` must all be 1.
    ``enable_internal_timers`` switches on event timers under the reference's timer names.
    ``block_aggregation`` selects the row-chunked aggregation (same result, bounded chunk size);
    ``overlap_aggregation`` requires it, as in the reference, and has nothing to overlap with on one
    GPU.  ``tune_gemms`` is accepted and ignored: the layout tuner of the reference chooses between
    transposed library calls, which does not apply to the hand-written kernels.
    """
    # overlap_aggregation can only be used with block_aggregation (plexus/plexus.py:32)
    assert not overlap_aggregation or block_aggregation
    if (G_intra_r, G_intra_c, G_intra_d) != (1, 1, 1):
        raise ValueError(
            "plexus_amd runs on one GPU: G_intra_r, G_intra_c and G_intra_d must be 1 (got %d x %d x %d)"
            % (G_intra_r, G_intra_c, G_intra_d)
        )
    global block_agg, overlap_agg, tune_gemm, _initialized
    block_agg, overlap_agg, tune_gemm = block_aggregation, overlap_aggregation, tune_gemms
    _timers.get_timers().enabled = bool(enable_internal_timers)
    _initialized = True
