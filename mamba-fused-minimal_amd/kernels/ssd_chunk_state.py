"""Stands in for the reference module kernels/ssd_chunk_state.py: ``_chunk_cumsum_fwd`` (:176-199) and
``_chunk_state_fwd`` (:202-232)."""
from ssd_amd.ops import _chunk_cumsum_fwd, _chunk_state_fwd

__all__ = ["_chunk_cumsum_fwd", "_chunk_state_fwd"]
