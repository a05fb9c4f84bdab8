"""Stands in for the reference module kernels/fused_concurrent.py (:255-331)."""
from ssd_amd.ops import _fused_chunk_state_state_passing_fwd_concurrent

__all__ = ["_fused_chunk_state_state_passing_fwd_concurrent"]
