"""Host-side mirror of the reference call surface for the SSD chunk-state + state-passing path.

Same names, positional order, defaults, shape asserts and output shapes/dtypes as
  kernels/ssd_chunk_state.py:202-232       _chunk_state_fwd
  kernels/ssd_state_passing.py:87-115      _state_passing_fwd
  kernels/fused_globalbar.py:201-266       _fused_chunk_state_state_passing_fwd_globalbar
  kernels/fused_concurrent.py:255-331      _fused_chunk_state_state_passing_fwd_concurrent
of the reference.  The wrappers own allocation and argument checking; the arithmetic runs in the gfx950 HIP
kernels behind the C ABI of libssd_gfx950.so, asynchronously on the current torch stream."""
import ctypes
import math
import threading

import torch

from . import _lib


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


# Workspaces of the ticket / flag-chain kernel that the wrappers keep to themselves: one per (device, stream), grown on
# demand, with the epoch of the last launch on it.  A workspace nobody else writes to lets a call tell the library that
# the launch before left it in order (ssd_fused_opts.epoch), which saves the fill launch in front of the kernel.
_WORKSPACES = {}                       # (device index, stream handle) -> _Kept
_WORKSPACES_LOCK = threading.Lock()    # guards the dictionary only; a launch holds its entry's own lock


class _Epochs:
    """The epochs of one kept workspace as ssd_fused_opts.epoch wants them: 0 for the first call (the library clears the
    workspace and counts the call as epoch 1), then 2, 3, ... -- but only calls that ran the chain kernel count, a failed
    call makes the contents unknown again, the count starts over before it could overflow, and a call that looks at
    more flags than the last clearing covered (more state tiles x chunks than the call that was given epoch 0) clears
    again: the flags beyond hold whatever the memory held before, possibly the value of the coming epoch."""
    LIMIT = 1 << 30

    def __init__(self):
        self.last = 0                      # epoch of the last chain launch on the workspace; 0 = contents unknown
        self.cleared = 0                   # (state tile, chunk) pairs whose flags the last clearing covered

    def next(self, pairs):
        if self.last >= self.LIMIT or pairs > self.cleared:
            self.last = 0
        return 0 if self.last == 0 else self.last + 1

    def done(self, epoch, rc, used_workspace, pairs):
        if rc:
            self.last = 0
            self.cleared = 0
        elif used_workspace:
            self.last = max(epoch, 1)
            if epoch <= 0:
                self.cleared = pairs


class _Kept:
    """A workspace the wrappers keep for one (device, stream), the epochs of the launches on it and the lock that
    keeps those launches in order (epochs must reach the stream in the order they were handed out)."""

    def __init__(self, tensor):
        self.tensor = tensor
        self.epochs = _Epochs()
        self.lock = threading.Lock()


def _workspace_key(device, stream=None):
    stream = torch.cuda.current_stream(device) if stream is None else stream
    return (device.index if device.index is not None else torch.cuda.current_device(), stream.cuda_stream)


def _own_workspace(x, nbytes):
    """-> the _Kept of x's device and current stream, holding at least nbytes (None under stream capture)."""
    if torch.cuda.is_current_stream_capturing():
        # a captured launch is replayed with the same arguments: the same epoch again and again would take the flags of
        # the replay before for its own.  Epoch 0 (clear every time) is what a graph needs.
        return None
    key = _workspace_key(x.device)
    with _WORKSPACES_LOCK:
        ent = _WORKSPACES.get(key)
        if ent is None or ent.tensor.numel() * 4 < nbytes:
            ent = _Kept(torch.empty((max(nbytes, 1 << 16) + 3) // 4, device=x.device, dtype=torch.int32))
            _WORKSPACES[key] = ent
    return ent


def release_workspaces():
    """Drops the workspaces the fused wrappers keep per (device, stream): a few hundred KB each as a rule, a quarter
    of an fp32 ``out`` after a call with bf16 passed states.  The next call allocates (and clears) a new one.  Launches
    already enqueued keep theirs alive through the caching allocator's stream ordering."""
    with _WORKSPACES_LOCK:
        _WORKSPACES.clear()


def _launch_on_own_workspace(x, nbytes, launch, used, pairs):
    """Runs launch(workspace, epoch) -> status on the wrappers' workspace for x's device and stream.  pairs: the
    (state tile, chunk) pairs of the call, i.e. the flags it looks at.  Only launches on the same device and stream
    wait for each other here."""
    ent = _own_workspace(x, nbytes)
    if ent is None:
        return launch(torch.empty(((nbytes + 3) // 4,), device=x.device, dtype=torch.int32), 0)
    with ent.lock:
        epoch = ent.epochs.next(pairs)
        rc = launch(ent.tensor, epoch)
        ent.epochs.done(epoch, rc, used.value, pairs)
        return rc


def fused_status(device=None, stream=None):
    """What the last fused call of this module on ``device`` and ``stream`` (defaults: the current ones) left in the
    workspace the wrappers keep for them: waits for the stream and returns 0, or the negative ssd_status of
    ssd_fused_workspace_status (-7 a flag wait ran out, -8 two XCDs drew from one counter, -9 a counter that owns work
    was never served, -10 the workspace was not what the epoch promised) -- the outputs of that call are then
    unusable.  Ask before the next fused call on the same stream, which starts the record afresh.  0 also when no call
    has used that workspace (another kernel family served it).  The reference's fused kernels have no such report:
    their spin loops are unbounded and a failure is a hang (kernels/fused_concurrent.py:11, 300)."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    stream = torch.cuda.current_stream(device) if stream is None else stream
    with _WORKSPACES_LOCK:
        ent = _WORKSPACES.get(_workspace_key(device, stream))
    if ent is None:
        return 0
    with ent.lock, torch.cuda.device(device):
        return int(_lib.load().ssd_fused_workspace_status(ctypes.c_void_p(ent.tensor.data_ptr()),
                                                          ctypes.c_void_p(stream.cuda_stream)))


def _prep_inputs(B, x, dt, dA_cumsum, seq_idx):
    # Callers guarantee a unit innermost stride for x and B (main.py:45-54 makes them contiguous otherwise).
    if x.stride(-1) != 1:
        x = x.contiguous()
    if B.stride(-1) != 1:
        B = B.contiguous()
    if B.dtype != x.dtype:
        B = B.to(x.dtype)
    if dt.dtype != torch.float32:
        dt = dt.float()
    if dA_cumsum.dtype != torch.float32:
        dA_cumsum = dA_cumsum.float()
    if seq_idx is not None and seq_idx.dtype != torch.int32:
        seq_idx = seq_idx.to(torch.int32)
    return B, x, dt, dA_cumsum, seq_idx


def _chunk_state_fwd(B, x, dt, dA_cumsum, seq_idx=None, states=None, states_in_fp32=True):
    return _chunk_state_impl(B, x, dt, dA_cumsum, seq_idx, states, states_in_fp32, True)


def _chunk_state_impl(B, x, dt, dA_cumsum, seq_idx, states, states_in_fp32, _clamp):
    # _clamp=False evaluates the decay as the reference's fused kernels do (no min(., 0), fused_globalbar.py:106)
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == dt.shape
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
    if states is not None:
        assert states.shape == (batch, nchunks, nheads, headdim, dstate)
    _lib.require_device(x, "_chunk_state_fwd")
    lib = _lib.load()
    if states is None:
        states_dtype = torch.float32 if states_in_fp32 else B.dtype
        states = torch.empty((batch, nchunks, nheads, headdim, dstate), device=x.device, dtype=states_dtype)
    B, x, dt, dA_cumsum, seq_idx = _prep_inputs(B, x, dt, dA_cumsum, seq_idx)
    dims = _lib.dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)
    with torch.cuda.device(x.device):
        rc = lib.ssd_chunk_state_fwd(_lib.tensor_arg(x), _lib.tensor_arg(B), _lib.tensor_arg(dt),
                                     _lib.tensor_arg(dA_cumsum), _lib.tensor_arg(seq_idx), _lib.tensor_arg(states),
                                     dims, 1 if _clamp else 0, _stream(x))
    _lib.check(rc, "ssd_chunk_state_fwd")
    return states


def _state_passing_fwd(states, dA_chunk_cumsum, initial_states=None, seq_idx=None, chunk_size=None,
                       out_dtype=None):
    batch, nchunks, nheads, dim = states.shape
    assert dA_chunk_cumsum.shape == (batch, nheads, nchunks)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, dim)
    seqlen = 0
    if seq_idx is not None:
        assert chunk_size is not None
        seqlen = seq_idx.shape[-1]
        assert seq_idx.shape == (batch, seqlen)
    _lib.require_device(states, "_state_passing_fwd")
    lib = _lib.load()
    out_dtype = states.dtype if out_dtype is None else out_dtype
    out = torch.empty((batch, nchunks, nheads, dim), device=states.device, dtype=out_dtype)
    final_states = torch.empty((batch, nheads, dim), device=states.device, dtype=torch.float32)
    if states.stride(-1) != 1:
        states = states.contiguous()
    if dA_chunk_cumsum.dtype != torch.float32:
        dA_chunk_cumsum = dA_chunk_cumsum.float()
    if initial_states is not None and initial_states.stride(-1) != 1:
        initial_states = initial_states.contiguous()
    if seq_idx is not None and seq_idx.dtype != torch.int32:
        seq_idx = seq_idx.to(torch.int32)
    with torch.cuda.device(states.device):
        rc = lib.ssd_state_passing_fwd(_lib.tensor_arg(states), _lib.tensor_arg(dA_chunk_cumsum),
                                       _lib.tensor_arg(initial_states), _lib.tensor_arg(seq_idx),
                                       _lib.tensor_arg(out), _lib.tensor_arg(final_states),
                                       batch, nchunks, nheads, dim, seqlen,
                                       chunk_size if seq_idx is not None else 0, _stream(states))
    _lib.check(rc, "ssd_state_passing_fwd")
    return out, final_states


def _fused_chunk_state_state_passing_fwd(B, x, dt, dA_cumsum, out_dtype, initial_states=None, seq_idx=None,
                                         states=None, states_in_fp32=True, _clamp=True, _kernel=0, _spin_limit=0,
                                         _workspace=None, _chunks_per_item=0, _epoch=0):
    """One launch for chunk state + state passing.  Returns (out (b,C,H,P,N) out_dtype, final_states (b,H,P,N) fp32).

    Unlike the reference's fused wrappers, the per-chunk states are an internal quantity that never reaches
    memory unless the caller passes a ``states=`` buffer, which is then filled as a side effect.

    The reference's wrappers allocate their counters per call (kernels/fused_globalbar.py:237-238,
    kernels/fused_concurrent.py:296-298); so does this one: a small int32 workspace for the ticket counter and the
    flags of the kernel that spreads a sequence's chunks over all compute units (plus, with bf16 ``out_dtype``, the
    fp32 copies of the states that cross between that kernel's work items).  ``_kernel`` (0 = let the library
    choose, 1 = insist on that kernel, 2 / 3 = and on its per-XCD / device-wide variant), ``_chunks_per_item``
    (1, 2 or 4 consecutive chunks per work item of that kernel, 0 = choose), ``_spin_limit`` (polls before a flag wait gives up, 0 = default) and
    ``_workspace`` (an int32 tensor to use instead of the wrapper's own, which it keeps per device and stream and whose
    fill launch it saves from the second call on) with ``_epoch`` (ssd_fused_opts.epoch for that tensor) are test and
    tuning hooks."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum.shape == dt.shape
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
    if states is not None:
        assert states.shape == (batch, nchunks, nheads, headdim, dstate)
        states_dtype = states.dtype
    else:
        states_dtype = torch.float32 if states_in_fp32 else B.dtype
    assert dA_cumsum.shape[:3] == (batch, nheads, nchunks)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, headdim, dstate)
    assert chunk_size is not None
    _lib.require_device(x, "_fused_chunk_state_state_passing_fwd")
    lib = _lib.load()
    out_dtype = states_dtype if out_dtype is None else out_dtype
    out = torch.empty((batch, nchunks, nheads, headdim, dstate), device=x.device, dtype=out_dtype)
    final_states = torch.empty((batch, nheads, headdim, dstate), device=x.device, dtype=torch.float32)
    B, x, dt, dA_cumsum, seq_idx = _prep_inputs(B, x, dt, dA_cumsum, seq_idx)
    if initial_states is not None and initial_states.stride(-1) != 1:
        initial_states = initial_states.contiguous()
    dims = _lib.dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)

    used = ctypes.c_int32(0)

    def launch(workspace, epoch):
        opts = _lib.SsdFusedOpts(workspace.data_ptr(), workspace.numel() * 4, int(_spin_limit), int(_kernel),
                                 int(_chunks_per_item), int(epoch), ctypes.pointer(used))
        with torch.cuda.device(x.device):
            return lib.ssd_fused_chunk_state_passing_fwd_ws(
                _lib.tensor_arg(x), _lib.tensor_arg(B), _lib.tensor_arg(dt), _lib.tensor_arg(dA_cumsum),
                _lib.tensor_arg(seq_idx), _lib.tensor_arg(initial_states), _lib.tensor_arg(states),
                _lib.tensor_arg(out), _lib.tensor_arg(final_states), dims, 1 if _clamp else 0, ctypes.byref(opts),
                _stream(x))

    if _workspace is not None:
        rc = launch(_workspace, _epoch)
    else:
        # bf16 passed states: the workspace also takes the fp32 states that cross between work items (a quarter of
        # an fp32 `out`, as a rule); 0 = that kernel is not offered for these arguments
        nbytes = 0
        if states is None:          # with a `states` buffer the call runs on other kernels anyway
            nbytes = int(lib.ssd_fused_workspace_bytes_for(dims, _lib._DTYPES.get(out_dtype, -1), int(_chunks_per_item)))
        rc = _launch_on_own_workspace(x, nbytes or int(lib.ssd_fused_workspace_bytes(dims)), launch, used,
                                      batch * nheads * ((headdim + 31) // 32) * nchunks)
    _lib.check(rc, "ssd_fused_chunk_state_passing_fwd_ws")
    return out, final_states


def _fused_chunk_state_state_passing_fwd_static(B, x, dt, dA_cumsum, out, final_states, initial_states=None, seq_idx=None,
                                                _clamp=True):
    """The fused call on the entry point that allocates nothing (ssd_fused_chunk_state_passing_fwd_static): the
    caller brings ``out`` (b,C,H,P,N) fp32 and ``final_states`` (b,H,P,N) fp32, the tickets and flags live in a
    fixed array inside the library, and this wrapper creates no tensor either (inputs must already have the types
    and unit inner strides the kernel takes).  No counterpart in the reference.  Calls that may overlap on one GPU
    race on that array."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, nheads, nchunks, chunk_size) and dA_cumsum.shape == dt.shape
    assert out.shape == (batch, nchunks, nheads, headdim, dstate) and final_states.shape == (batch, nheads, headdim, dstate)
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen) and seq_idx.dtype == torch.int32
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, headdim, dstate)
    _lib.require_device(x, "_fused_chunk_state_state_passing_fwd_static")
    lib = _lib.load()
    dims = _lib.dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)
    with torch.cuda.device(x.device):
        rc = lib.ssd_fused_chunk_state_passing_fwd_static(
            _lib.tensor_arg(x), _lib.tensor_arg(B), _lib.tensor_arg(dt), _lib.tensor_arg(dA_cumsum),
            _lib.tensor_arg(seq_idx), _lib.tensor_arg(initial_states), _lib.tensor_arg(out),
            _lib.tensor_arg(final_states), dims, 1 if _clamp else 0, _stream(x))
    _lib.check(rc, "ssd_fused_chunk_state_passing_fwd_static")
    return out, final_states


def _fused_static_status(device=None):
    """Waits for the current stream and returns 0, or -7 if a flag wait of the last
    ssd_fused_chunk_state_passing_fwd_static launch on this device ran out."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    with torch.cuda.device(device):
        return int(_lib.load().ssd_fused_static_status(ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)))


def _fused_workspace_status(workspace):
    """Waits for the current stream and returns 0, or the negative status of the last fused launch that used
    ``workspace`` (ssd_fused_workspace_status: -7 ... -10)."""
    with torch.cuda.device(workspace.device):
        return int(_lib.load().ssd_fused_workspace_status(ctypes.c_void_p(workspace.data_ptr()), _stream(workspace)))


def fused_plan(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, workspace=True, compute_units=0):
    """Which kernel family the fused call would run on plain bf16 / fp32 tensors of these sizes and the library's
    estimate of every family's duration (no counterpart in the reference, whose fused wrappers have one kernel each:
    kernels/fused_globalbar.py:201-266, kernels/fused_concurrent.py:255-331).  Host logic only: needs no GPU.
    Returns {"family": name, "chunks_per_item": R or 0, "estimate_us": {name: microseconds or None}}."""
    nchunks = (seqlen + chunk_size - 1) // chunk_size
    dims = _lib.dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)
    plan = _lib.SsdFusedPlan()
    _lib.check(_lib.load().ssd_query_fused_plan(dims, 1 if workspace else 0, int(compute_units), ctypes.byref(plan)),
               "ssd_query_fused_plan")
    return {"family": _lib.SSD_FAMILIES[plan.family], "chunks_per_item": int(plan.chunks_per_item),
            "estimate_us": {n: (float(v) if v > 0 else None) for n, v in zip(_lib.SSD_FAMILIES, plan.estimate_us)}}


def _fused_chunk_state_state_passing_fwd_globalbar(B, x, dt, dA_cumsum, out_dtype, initial_states=None,
                                                   seq_idx=None, states=None, states_in_fp32=True):
    """Drop-in for kernels/fused_globalbar.py:201 (same signature and returns)."""
    return _fused_chunk_state_state_passing_fwd(B, x, dt, dA_cumsum, out_dtype, initial_states=initial_states,
                                                seq_idx=seq_idx, states=states, states_in_fp32=states_in_fp32)


def _fused_chunk_state_state_passing_fwd_concurrent(B, x, dt, dA_cumsum, out_dtype, initial_states=None,
                                                    seq_idx=None, states=None, states_in_fp32=True):
    """Drop-in for kernels/fused_concurrent.py:255 (same signature and returns; prints nothing)."""
    return _fused_chunk_state_state_passing_fwd(B, x, dt, dA_cumsum, out_dtype, initial_states=initial_states,
                                                seq_idx=seq_idx, states=states, states_in_fp32=states_in_fp32)


def _chunk_cumsum_fwd(dt, A, chunk_size, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """dt preparation + per-chunk cumulative sum of dt * A; same call surface as the reference's
    kernels/ssd_chunk_state.py:176-199.  dt (batch, seqlen, nheads) -> (dA_cumsum, dt_out), both
    (batch, nheads, nchunks, chunk_size) fp32."""
    batch, seqlen, nheads = dt.shape
    assert A.shape == (nheads,)
    if dt_bias is not None:
        assert dt_bias.shape == (nheads,)
    _lib.require_device(dt, "_chunk_cumsum_fwd")
    nchunks = math.ceil(seqlen / chunk_size)
    dt_out = torch.empty(batch, nheads, nchunks, chunk_size, device=dt.device, dtype=torch.float32)
    dA_cumsum = torch.empty(batch, nheads, nchunks, chunk_size, device=dt.device, dtype=torch.float32)
    lib = _lib.load()
    with torch.cuda.device(dt.device):
        rc = lib.ssd_chunk_cumsum_fwd(_lib.tensor_arg(dt), _lib.tensor_arg(A), _lib.tensor_arg(dt_bias),
                                      _lib.tensor_arg(dt_out), _lib.tensor_arg(dA_cumsum), batch, seqlen, nheads,
                                      int(chunk_size), int(bool(dt_softplus)), float(dt_limit[0]), float(dt_limit[1]),
                                      _stream(dt))
    _lib.check(rc, "ssd_chunk_cumsum_fwd")
    return dA_cumsum, dt_out


def _fused_cumsum_chunk_state_state_passing_fwd(B, x, dt, A, chunk_size, out_dtype, dt_bias=None, dt_softplus=False,
                                                dt_limit=(0.0, float("inf")), initial_states=None, seq_idx=None,
                                                _clamp=True, _kernel=0, _chunks_per_item=0, _workspace=None):
    """``_chunk_cumsum_fwd`` followed by ``_fused_chunk_state_state_passing_fwd`` in one call (the first three stages of
    the reference's main.py:78-100): dt is the raw (batch, seqlen, nheads) tensor.  Returns
    (out (b,C,H,P,N) out_dtype, final_states (b,H,P,N) fp32, dA_cumsum, dt_out (b,H,C,Q) fp32).

    Two launches; where the library runs its ticket / flag-chain kernel, the first one clears that kernel's workspace
    on its way.  ``_kernel``, ``_chunks_per_item`` and ``_workspace`` are the hooks of
    ``_fused_chunk_state_state_passing_fwd``."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, seqlen, nheads)
    assert A.shape == (nheads,)
    if dt_bias is not None:
        assert dt_bias.shape == (nheads,)
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
        if seq_idx.dtype != torch.int32:
            seq_idx = seq_idx.to(torch.int32)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, headdim, dstate)
        if initial_states.stride(-1) != 1:
            initial_states = initial_states.contiguous()
    _lib.require_device(x, "_fused_cumsum_chunk_state_state_passing_fwd")
    nchunks = math.ceil(seqlen / chunk_size)
    if x.stride(-1) != 1:
        x = x.contiguous()
    if B.stride(-1) != 1:
        B = B.contiguous()
    dt_out = torch.empty(batch, nheads, nchunks, chunk_size, device=x.device, dtype=torch.float32)
    dA_cumsum = torch.empty(batch, nheads, nchunks, chunk_size, device=x.device, dtype=torch.float32)
    out = torch.empty((batch, nchunks, nheads, headdim, dstate), device=x.device, dtype=out_dtype or torch.float32)
    final_states = torch.empty((batch, nheads, headdim, dstate), device=x.device, dtype=torch.float32)
    dims = _lib.dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)
    T = _lib.tensor_arg
    lib = _lib.load()

    used = ctypes.c_int32(0)

    def launch(workspace, epoch):
        opts = _lib.SsdFusedOpts(workspace.data_ptr(), workspace.numel() * 4, 0, int(_kernel), int(_chunks_per_item), int(epoch),
                                 ctypes.pointer(used))
        with torch.cuda.device(x.device):
            return lib.ssd_fused_cumsum_chunk_state_passing_fwd_ws(
                T(x), T(B), T(dt), T(A), T(dt_bias), T(seq_idx), T(initial_states), T(dt_out), T(dA_cumsum), T(out),
                T(final_states), dims, int(bool(dt_softplus)), float(dt_limit[0]), float(dt_limit[1]), 1 if _clamp else 0,
                ctypes.byref(opts), _stream(x))

    if _workspace is not None:
        rc = launch(_workspace, 0)
    else:
        nbytes = int(lib.ssd_fused_workspace_bytes_for(dims, _lib._DTYPES.get(out.dtype, -1), int(_chunks_per_item)))
        rc = _launch_on_own_workspace(x, nbytes or int(lib.ssd_fused_workspace_bytes(dims)), launch, used,
                                      batch * nheads * ((headdim + 31) // 32) * nchunks)
    _lib.check(rc, "ssd_fused_cumsum_chunk_state_passing_fwd_ws")
    return out, final_states, dA_cumsum, dt_out


def _chunk_scan_states_fwd(C, prev_states, dA_cumsum, seq_idx=None, out=None, out_dtype=None, accumulate=False):
    """The state-consuming half of the reference's ``_chunk_scan_fwd`` (kernels/ssd_chunk_scan.py:94-117, wrapper
    :172-224): y[b,cQ+m,h,:] = scale_m * (C[b,cQ+m,g,:] . prev_states[b,c,h]), scale_m = exp(dA_cumsum[b,h,c,m]) where
    seq_idx[b,cQ+m] equals seq_idx[b,cQ-1] (0 for the first chunk) and 0 elsewhere.

    C (batch, seqlen, ngroups, dstate); prev_states (batch, nchunks, nheads, headdim, dstate), the ``out`` of the
    state passing; dA_cumsum (batch, nheads, nchunks, chunk_size).  Returns y (batch, seqlen, nheads, headdim) of
    ``out_dtype`` (default: C's, as the reference's ``out`` takes x's); with ``out=`` the result goes there, and with
    ``accumulate=True`` it is added to what ``out`` holds (the intra-chunk half of the scan)."""
    batch, seqlen, ngroups, dstate = C.shape
    _, nchunks, nheads, headdim, _ = prev_states.shape
    chunk_size = dA_cumsum.shape[-1]
    assert nheads % ngroups == 0
    assert prev_states.shape == (batch, nchunks, nheads, headdim, dstate)
    assert dA_cumsum.shape == (batch, nheads, nchunks, chunk_size)
    assert nchunks == math.ceil(seqlen / chunk_size)
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
        if seq_idx.dtype != torch.int32:
            seq_idx = seq_idx.to(torch.int32)
    _lib.require_device(C, "_chunk_scan_states_fwd")
    if out is None:
        assert not accumulate, "accumulate=True needs the tensor to add to (out=)"
        out = torch.empty(batch, seqlen, nheads, headdim, device=C.device, dtype=out_dtype or C.dtype)
    else:
        assert out.shape == (batch, seqlen, nheads, headdim) and out.stride(-1) == 1
    if C.stride(-1) != 1:
        C = C.contiguous()
    if prev_states.stride(-1) != 1:
        prev_states = prev_states.contiguous()
    if dA_cumsum.dtype != torch.float32:
        dA_cumsum = dA_cumsum.float()
    dims = _lib.dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)
    with torch.cuda.device(C.device):
        rc = _lib.load().ssd_chunk_scan_states_fwd(_lib.tensor_arg(C), _lib.tensor_arg(prev_states),
                                                   _lib.tensor_arg(dA_cumsum), _lib.tensor_arg(seq_idx),
                                                   _lib.tensor_arg(out), dims, int(bool(accumulate)), _stream(C))
    _lib.check(rc, "ssd_chunk_scan_states_fwd")
    return out


def _fused_chunk_state_state_passing_scan_fwd(B, x, C, dt, dA_cumsum, out_dtype=torch.float32, initial_states=None,
                                              seq_idx=None, y=None, y_dtype=None, accumulate=False, return_states=True,
                                              _clamp=True, _kernel=0, _chunks_per_item=0, _workspace=None, _epoch=0,
                                              _spin_limit=0):
    """Chunk state + state passing + the state-dependent half of the chunk scan in one call
    (ssd_fused_chunk_state_passing_scan_fwd): what the reference does with kernels/fused_concurrent.py:255-331 followed
    by the state half of kernels/ssd_chunk_scan.py:94-117 (main.py:100-101).  Returns (out or None, final_states, y).

    ``return_states=False`` leaves ``out`` -- (b,C,H,P,N), the state entering every chunk -- out altogether: where the
    ticket / flag-chain kernel serves the call the passed states then never reach memory.  ``y`` (b,L,H,P) is created in
    ``y_dtype`` (default C's, as the reference's scan output takes x's) unless given; ``accumulate=True`` adds to a given
    ``y`` (the intra-chunk half of the scan computed elsewhere).  The other arguments are those of
    ``_fused_chunk_state_state_passing_fwd``."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate) and C.shape == B.shape
    assert dt.shape == (batch, nheads, nchunks, chunk_size) and dA_cumsum.shape == dt.shape
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, headdim, dstate)
    _lib.require_device(x, "_fused_chunk_state_state_passing_scan_fwd")
    lib = _lib.load()
    if y is None:
        assert not accumulate, "accumulate=True needs the tensor to add to (y=)"
        y = torch.empty(batch, seqlen, nheads, headdim, device=x.device, dtype=y_dtype or C.dtype)
    else:
        assert y.shape == (batch, seqlen, nheads, headdim) and y.stride(-1) == 1
    B, x, dt, dA_cumsum, seq_idx = _prep_inputs(B, x, dt, dA_cumsum, seq_idx)
    if C.stride(-1) != 1:
        C = C.contiguous()
    if initial_states is not None and initial_states.stride(-1) != 1:
        initial_states = initial_states.contiguous()
    final_states = torch.empty((batch, nheads, headdim, dstate), device=x.device, dtype=torch.float32)
    dims = _lib.dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)
    T = _lib.tensor_arg
    pairs = batch * nheads * ((headdim + 31) // 32) * nchunks
    used = ctypes.c_int32(0)

    def call(out):
        def launch(workspace, epoch):
            opts = _lib.SsdFusedOpts(workspace.data_ptr(), workspace.numel() * 4, int(_spin_limit), int(_kernel),
                                     int(_chunks_per_item), int(epoch), ctypes.pointer(used))
            with torch.cuda.device(x.device):
                return lib.ssd_fused_chunk_state_passing_scan_fwd(
                    T(x), T(B), T(C), T(dt), T(dA_cumsum), T(seq_idx), T(initial_states), T(out), T(final_states), T(y),
                    dims, 1 if _clamp else 0, int(bool(accumulate)), ctypes.byref(opts), _stream(x))

        if _workspace is not None:
            return launch(_workspace, _epoch)
        nbytes = int(lib.ssd_fused_scan_workspace_bytes(dims, 1 if out is not None else 0, int(_chunks_per_item)))
        return _launch_on_own_workspace(x, nbytes, launch, used, pairs)

    out = None
    if return_states:
        out = torch.empty((batch, nchunks, nheads, headdim, dstate), device=x.device, dtype=out_dtype or torch.float32)
    rc = call(out)
    if rc == _lib.SSD_ERR_SCRATCH and out is None and _kernel == 0:
        # arguments the one-launch kernel does not take: the passed states then need a place, which this wrapper (the
        # owner of all allocations) provides and drops again
        rc = call(torch.empty((batch, nchunks, nheads, headdim, dstate), device=x.device, dtype=torch.float32))
    _lib.check(rc, "ssd_fused_chunk_state_passing_scan_fwd")
    return out, final_states, y


def set_scan_kernel(kernel):
    """Tuning / test hook (no counterpart in the reference): 1 = the scan consumer runs one workgroup per head, 2 = one
    workgroup per run of heads wherever that kernel applies, 0 = let the library choose.  Returns the previous setting."""
    rc = _lib.load().ssd_set_scan_kernel(int(kernel))
    if rc < 0:
        raise ValueError("scan kernel must be 0, 1 or 2")
    return rc


def measure_traffic_floor(B, x, dt, dA_cumsum, out, final_states, part=0):
    """Measurement hook (no counterpart in the reference): enqueues the kernel that moves the bytes of the fused call on
    these tensors -- x and B read, one fp32 state tile per (state tile, chunk) written -- and does nothing else
    (ssd_measure_traffic_floor[_part]).  ``out`` (b,C,H,P,N) fp32 is overwritten with zeros.  ``part``: 0 = loads and
    stores, 1 = the loads only (``out`` is left alone), 2 = the stores only."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert out.shape == (batch, nchunks, nheads, headdim, dstate) and final_states.shape == (batch, nheads, headdim, dstate)
    _lib.require_device(x, "measure_traffic_floor")
    dims = _lib.dims_arg(batch, seqlen, nheads, headdim, dstate, ngroups, chunk_size, nchunks)
    T = _lib.tensor_arg
    with torch.cuda.device(x.device):
        rc = _lib.load().ssd_measure_traffic_floor_part(T(x), T(B), T(dt), T(dA_cumsum), T(out), T(final_states), dims, int(part),
                                                        _stream(x))
    _lib.check(rc, "ssd_measure_traffic_floor_part")


def set_chain_xcds(xcds):
    """Test hook (no counterpart in the reference): the number of XCDs the per-XCD variant of the ticket / flag-chain
    kernel deals its units to; 0 = from the device.  A wrong count provokes the kernel's own checks
    (fused_status -8 / -9).  Returns the previous setting."""
    rc = _lib.load().ssd_set_chain_xcds(int(xcds))
    if rc < 0:
        raise ValueError("the number of XCDs must be 0 (from the device) .. 16")
    return rc


def set_segment_chunks(chunks):
    """Tuning / test hook (no counterpart in the reference): consecutive chunks per workgroup when the kernel with
    four tiles per workgroup serves ``_chunk_state_fwd``; 0 = let the library choose.  Returns the previous setting."""
    rc = _lib.load().ssd_set_segment_chunks(int(chunks))
    if rc < 0:
        raise ValueError("chunks per workgroup must be 0 (automatic) or positive")
    return rc


def set_token_split(waves):
    """Tuning / test hook (no counterpart in the reference): 2 or 4 = the token-split bf16 MFMA kernels with that
    many waves per state tile, 1 = the kernel with one wave per tile and four tiles per workgroup wherever it
    applies, 0 = let the library choose.  While it is not 0 the library does not pick the ticket / flag-chain kernel by
    itself either.  Returns the previous setting."""
    rc = _lib.load().ssd_set_token_split(int(waves))
    if rc < 0:
        raise ValueError("token split must be 0, 1, 2 or 4")
    return rc
