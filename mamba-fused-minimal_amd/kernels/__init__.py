"""Module names of the reference's ``kernels`` package, for callers that only swap the import root:
``from kernels.ssd_chunk_state import _chunk_state_fwd`` etc. resolve to the gfx950 implementation."""
