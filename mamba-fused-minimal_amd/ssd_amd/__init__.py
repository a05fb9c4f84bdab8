"""MI355X (gfx950) implementation of the Mamba2 SSD chunk-state + state-passing path.

Host wrappers with the reference's call surface over hand-written HIP kernels (libssd_gfx950.so, C ABI in
include/ssd_gfx950.h)."""
from .ops import (_chunk_cumsum_fwd, _fused_cumsum_chunk_state_state_passing_fwd, _chunk_scan_states_fwd, _chunk_state_fwd, _state_passing_fwd, _fused_chunk_state_state_passing_fwd,
                  _fused_chunk_state_state_passing_fwd_globalbar, _fused_chunk_state_state_passing_fwd_concurrent, set_scan_kernel, set_segment_chunks, set_token_split, _fused_workspace_status,
                  _fused_chunk_state_state_passing_fwd_static, _fused_static_status, fused_plan, release_workspaces, fused_status, set_chain_xcds, measure_traffic_floor, _fused_chunk_state_state_passing_scan_fwd)

__all__ = ["_chunk_cumsum_fwd", "_fused_cumsum_chunk_state_state_passing_fwd", "_chunk_scan_states_fwd", "_chunk_state_fwd", "_state_passing_fwd", "_fused_chunk_state_state_passing_fwd",
           "_fused_chunk_state_state_passing_fwd_globalbar", "_fused_chunk_state_state_passing_fwd_concurrent", "set_scan_kernel", "set_segment_chunks", "set_token_split", "_fused_workspace_status",
           "_fused_chunk_state_state_passing_fwd_static", "_fused_static_status", "fused_plan", "release_workspaces", "fused_status", "set_chain_xcds", "measure_traffic_floor", "_fused_chunk_state_state_passing_scan_fwd"]
