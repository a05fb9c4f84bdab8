"""Stands in for the reference module kernels/ssd_state_passing.py (:87-115)."""
from ssd_amd.ops import _state_passing_fwd

__all__ = ["_state_passing_fwd"]
