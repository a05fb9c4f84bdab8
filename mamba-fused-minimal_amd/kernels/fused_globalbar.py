"""Stands in for the reference module kernels/fused_globalbar.py (:201-266)."""
from ssd_amd.ops import _fused_chunk_state_state_passing_fwd_globalbar

__all__ = ["_fused_chunk_state_state_passing_fwd_globalbar"]
