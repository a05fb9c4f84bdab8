"""Stands in for the state-consuming half of the reference module kernels/ssd_chunk_scan.py: the contribution of the
state entering each chunk to ``_chunk_scan_fwd``'s output (:94-117).  The intra-chunk half (:119-169) is not part of
this library."""
from ssd_amd.ops import _chunk_scan_states_fwd

__all__ = ["_chunk_scan_states_fwd"]
