"""ctypes binding of libssd_gfx950.so (declared in include/ssd_gfx950.h).

There is no fallback: if the library is missing, or the tensors are not on a gfx950 device, the calls raise."""
import ctypes
import os

import torch

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_ROOT, "libssd_gfx950.so")

SSD_F32, SSD_BF16, SSD_F16 = 0, 1, 2
_DTYPES = {torch.float32: SSD_F32, torch.bfloat16: SSD_BF16, torch.float16: SSD_F16}

EXPORTS = ("ssd_version", "ssd_status_string", "ssd_chunk_state_fwd", "ssd_state_passing_fwd",
           "ssd_fused_chunk_state_passing_fwd", "ssd_fused_chunk_state_passing_fwd_ws", "ssd_fused_workspace_bytes", "ssd_fused_workspace_bytes_for",
           "ssd_fused_workspace_status", "ssd_fused_workspace_status_of", "ssd_set_chain_xcds", "ssd_measure_traffic_floor", "ssd_measure_traffic_floor_part", "ssd_fused_scan_workspace_bytes", "ssd_fused_chunk_state_passing_scan_fwd", "ssd_fused_chunk_state_passing_fwd_static", "ssd_fused_static_status",
           "ssd_fused_cumsum_chunk_state_passing_fwd", "ssd_fused_cumsum_chunk_state_passing_fwd_ws", "ssd_query_path", "ssd_query_fused_plan", "ssd_chunk_cumsum_fwd", "ssd_chunk_scan_states_fwd", "ssd_set_scan_kernel", "ssd_set_token_split", "ssd_set_segment_chunks")


class SsdTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("stride", ctypes.c_int64 * 5)]


class SsdDims(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in
                ("batch", "seqlen", "nheads", "headdim", "dstate", "ngroups", "chunk_size", "nchunks")]


class SsdFusedOpts(ctypes.Structure):
    _fields_ = [("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_uint64), ("spin_limit", ctypes.c_int32),
                ("kernel", ctypes.c_int32), ("chunks_per_item", ctypes.c_int32), ("epoch", ctypes.c_int32), ("used_workspace", ctypes.POINTER(ctypes.c_int32))]


class SsdFusedPlan(ctypes.Structure):
    _fields_ = [("family", ctypes.c_int32), ("chunks_per_item", ctypes.c_int32), ("estimate_us", ctypes.c_float * 5)]


SSD_FAMILIES = ("generic", "token_split", "four_tile", "pair", "chain")
SSD_KERNEL_AUTO, SSD_KERNEL_CHAIN, SSD_KERNEL_CHAIN_LOCAL, SSD_KERNEL_CHAIN_GLOBAL = 0, 1, 2, 3
SSD_ERR_SCRATCH, SSD_ERR_CHAIN_TIMEOUT, SSD_ERR_CHAIN_XCD, SSD_ERR_CHAIN_INCOMPLETE, SSD_ERR_CHAIN_WORKSPACE = -6, -7, -8, -9, -10
SSD_WORKSPACE_HEADER_INTS = 128

_lib = None


def load():
    """Loads the shared library once.  Raises if it has not been built (python build.py)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python {os.path.join(_PKG_ROOT, 'build.py')}`; "
                          "there is no CPU or PyTorch fallback for this path")
    lib = ctypes.CDLL(LIB_PATH)
    T, D, vp, i32 = ctypes.POINTER(SsdTensor), ctypes.POINTER(SsdDims), ctypes.c_void_p, ctypes.c_int32
    lib.ssd_version.restype = ctypes.c_int
    lib.ssd_version.argtypes = []
    lib.ssd_status_string.restype = ctypes.c_char_p
    lib.ssd_status_string.argtypes = [ctypes.c_int]
    lib.ssd_chunk_state_fwd.restype = ctypes.c_int
    lib.ssd_chunk_state_fwd.argtypes = [T, T, T, T, T, T, D, ctypes.c_int, vp]
    lib.ssd_state_passing_fwd.restype = ctypes.c_int
    lib.ssd_state_passing_fwd.argtypes = [T, T, T, T, T, T, i32, i32, i32, i32, i32, i32, vp]
    lib.ssd_fused_chunk_state_passing_fwd.restype = ctypes.c_int
    lib.ssd_fused_chunk_state_passing_fwd.argtypes = [T, T, T, T, T, T, T, T, T, D, ctypes.c_int, vp]
    lib.ssd_fused_chunk_state_passing_fwd_ws.restype = ctypes.c_int
    lib.ssd_fused_chunk_state_passing_fwd_ws.argtypes = [T, T, T, T, T, T, T, T, T, D, ctypes.c_int, ctypes.POINTER(SsdFusedOpts), vp]
    lib.ssd_fused_workspace_bytes.restype = ctypes.c_uint64
    lib.ssd_fused_workspace_bytes.argtypes = [D]
    lib.ssd_fused_workspace_bytes_for.restype = ctypes.c_uint64
    lib.ssd_fused_workspace_bytes_for.argtypes = [D, ctypes.c_int, ctypes.c_int]
    lib.ssd_fused_workspace_status.restype = ctypes.c_int
    lib.ssd_fused_workspace_status.argtypes = [vp, vp]
    lib.ssd_fused_workspace_status_of.restype = ctypes.c_int
    lib.ssd_fused_workspace_status_of.argtypes = [ctypes.POINTER(ctypes.c_int32)]
    lib.ssd_fused_scan_workspace_bytes.restype = ctypes.c_uint64
    lib.ssd_fused_scan_workspace_bytes.argtypes = [D, ctypes.c_int, ctypes.c_int]
    lib.ssd_fused_chunk_state_passing_scan_fwd.restype = ctypes.c_int
    lib.ssd_fused_chunk_state_passing_scan_fwd.argtypes = [T] * 10 + [D, ctypes.c_int, ctypes.c_int, ctypes.POINTER(SsdFusedOpts), vp]
    lib.ssd_measure_traffic_floor.restype = ctypes.c_int
    lib.ssd_measure_traffic_floor.argtypes = [T, T, T, T, T, T, D, vp]
    lib.ssd_measure_traffic_floor_part.restype = ctypes.c_int
    lib.ssd_measure_traffic_floor_part.argtypes = [T, T, T, T, T, T, D, ctypes.c_int, vp]
    lib.ssd_set_chain_xcds.restype = ctypes.c_int
    lib.ssd_set_chain_xcds.argtypes = [ctypes.c_int]
    lib.ssd_fused_chunk_state_passing_fwd_static.restype = ctypes.c_int
    lib.ssd_fused_chunk_state_passing_fwd_static.argtypes = [T, T, T, T, T, T, T, T, D, ctypes.c_int, vp]
    lib.ssd_fused_static_status.restype = ctypes.c_int
    lib.ssd_fused_static_status.argtypes = [vp]
    lib.ssd_fused_cumsum_chunk_state_passing_fwd.restype = ctypes.c_int
    lib.ssd_fused_cumsum_chunk_state_passing_fwd.argtypes = [T] * 11 + [D, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int, vp]
    lib.ssd_fused_cumsum_chunk_state_passing_fwd_ws.restype = ctypes.c_int
    lib.ssd_fused_cumsum_chunk_state_passing_fwd_ws.argtypes = [T] * 11 + [D, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.POINTER(SsdFusedOpts), vp]
    lib.ssd_query_path.restype = ctypes.c_int
    lib.ssd_query_path.argtypes = [T, T, D]
    lib.ssd_query_fused_plan.restype = ctypes.c_int
    lib.ssd_query_fused_plan.argtypes = [D, ctypes.c_int, ctypes.c_int, ctypes.POINTER(SsdFusedPlan)]
    lib.ssd_chunk_cumsum_fwd.restype = ctypes.c_int
    lib.ssd_chunk_cumsum_fwd.argtypes = [T, T, T, T, T, i32, i32, i32, i32, ctypes.c_int, ctypes.c_float, ctypes.c_float, vp]
    lib.ssd_chunk_scan_states_fwd.restype = ctypes.c_int
    lib.ssd_chunk_scan_states_fwd.argtypes = [T, T, T, T, T, D, ctypes.c_int, vp]
    lib.ssd_set_scan_kernel.restype = ctypes.c_int
    lib.ssd_set_scan_kernel.argtypes = [ctypes.c_int]
    lib.ssd_set_token_split.restype = ctypes.c_int
    lib.ssd_set_token_split.argtypes = [ctypes.c_int]
    lib.ssd_set_segment_chunks.restype = ctypes.c_int
    lib.ssd_set_segment_chunks.argtypes = [ctypes.c_int]
    _lib = lib
    return lib


def tensor_arg(t):
    """ssd_tensor for a torch tensor (None -> a struct with a NULL data pointer)."""
    s = SsdTensor()
    if t is None:
        s.data = None
        return s
    if t.dtype == torch.int32:
        s.dtype = 0
    elif t.dtype in _DTYPES:
        s.dtype = _DTYPES[t.dtype]
    else:
        raise TypeError(f"unsupported dtype {t.dtype}")
    s.data = t.data_ptr()
    for i, st in enumerate(t.stride()):
        s.stride[i] = st
    return s


def dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks):
    return SsdDims(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)


def check(rc, what):
    if rc != 0:
        msg = load().ssd_status_string(rc).decode()
        raise RuntimeError(f"{what} failed: {msg} (status {rc})")


def require_device(t, what):
    if not t.is_cuda:
        raise RuntimeError(f"{what}: tensors must live on a gfx950 (MI355X) device; there is no CPU path")
