"""plexus_amd -- the GCN-layer hot path of Plexus as hand-written gfx950 kernels.

The Python surface keeps the reference's names (``plexus.init``, ``GCNConv``,
``parallel_cross_entropy``); the arithmetic runs in ``libplexus_hip.so`` through the C ABI of
``include/plexus_hip.h``.  One GPU, no collectives.
"""
from . import plexus  # noqa: F401
from .plexus import init  # noqa: F401

__all__ = ["init", "plexus"]
