"""Stands in for the reference module kernels/ssd_chunk_state.py (the ``_chunk_state_fwd`` half, :202-232)."""
from ssd_amd.ops import _chunk_state_fwd

__all__ = ["_chunk_state_fwd"]
