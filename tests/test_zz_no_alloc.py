"""GPU test of the entry point that allocates nothing (ssd_fused_chunk_state_passing_fwd_static), through the C ABI:
its outputs against those of ssd_fused_chunk_state_passing_fwd_ws on the same inputs -- the same kernel with a
caller-provided workspace --, on two calls in a row, the second with a smaller input, and against the CPU oracle
(rtol 2e-3 / atol 1e-3).  Collected last: the scratch array is shared by every call of the process."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev(t):
    return None if t is None else t.cuda()


def _pair(ops, oracle, kw, name):
    d = oracle.make_inputs(2, **kw)
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    init, seq = _dev(d["initial_states"]), _dev(d["seq_idx"])
    b, L, H, P = d["x"].shape
    N, C = d["B"].shape[-1], d["dt"].shape[2]
    print(f"[{name}] x{tuple(d['x'].shape)} chunks={C} init={init is not None} seq={seq is not None}", flush=True)
    # outputs poisoned: every element must be written by the call
    out = torch.full((b, C, H, P, N), float("nan"), device="cuda")
    fin = torch.full((b, H, P, N), float("nan"), device="cuda")
    ops._fused_chunk_state_state_passing_fwd_static(*args, out, fin, initial_states=init, seq_idx=seq)
    assert ops._fused_static_status() == 0
    want_out, want_fin = ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, initial_states=init, seq_idx=seq,
                                                                  _kernel=1)
    torch.cuda.synchronize()
    # the same kernel on the same inputs: the same bits
    assert torch.equal(out, want_out), f"{name}: out differs, max {float((out - want_out).abs().max()):.3e}"
    assert torch.equal(fin, want_fin), f"{name}: final_states differ"
    ref_out, ref_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"],
                                        seq_idx=d["seq_idx"])
    for got, want in ((out, ref_out), (fin, ref_fin)):
        err = (got.cpu() - want).abs()
        assert int((err > 1e-3 + 2e-3 * want.abs()).sum()) == 0, f"{name}: max abs err {float(err.max()):.3e}"


def test_static_scratch_entry_point_two_calls(oracle):
    import ssd_amd
    from ssd_amd import _lib
    _lib.load()
    assert torch.cuda.is_available(), "this test needs the MI355X"
    _pair(ssd_amd, oracle, dict(b=2, L=8192, H=16), "static.first")                  # 32 chunks, initial states
    _pair(ssd_amd, oracle, dict(b=1, L=2000, H=8, nseq=3), "static.second.smaller")  # fewer, ragged, packed sequences


def test_static_scratch_rejects_what_does_not_fit():
    from ssd_amd import _lib
    lib = _lib.load()
    # 262 144 ints: the header (128) plus one flag per (state tile, chunk).  b=8 L=131072 H=128 would need 1 M of them.
    # The call is rejected before anything is launched, so the tensors only need plausible descriptions.
    b, L, H, P, N, G, Q, C = 8, 131072, 128, 64, 128, 8, 256, 512
    dims = _lib.dims_arg(b, L, H, P, N, G, Q, C)
    assert lib.ssd_fused_workspace_bytes(dims) > 4 * (1 << 18)
    anchor = torch.zeros(64, device="cuda")

    def described(dtype, shape):
        t = _lib.SsdTensor()
        t.data = anchor.data_ptr()
        t.dtype = dtype
        stride = 1
        for i in reversed(range(len(shape))):
            t.stride[i] = stride
            stride *= shape[i]
        return t

    none = _lib.tensor_arg(None)
    rc = lib.ssd_fused_chunk_state_passing_fwd_static(
        described(_lib.SSD_BF16, (b, L, H, P)), described(_lib.SSD_BF16, (b, L, G, N)), described(_lib.SSD_F32, (b, H, C, Q)),
        described(_lib.SSD_F32, (b, H, C, Q)), none, none, described(_lib.SSD_F32, (b, C, H, P, N)),
        described(_lib.SSD_F32, (b, H, P, N)), dims, 1, None)
    assert rc == _lib.SSD_ERR_SCRATCH, rc
    assert "workspace" in lib.ssd_status_string(rc).decode()
    # bf16 passed states: the chain kernel would keep fp32 copies of them in its workspace, for which the array has no
    # room -- a shape this entry point does not cover, whatever the size
    b, L, C = 1, 1024, 4
    small = _lib.dims_arg(b, L, H, P, N, G, Q, C)
    rc = lib.ssd_fused_chunk_state_passing_fwd_static(
        described(_lib.SSD_BF16, (b, L, H, P)), described(_lib.SSD_BF16, (b, L, G, N)), described(_lib.SSD_F32, (b, H, C, Q)),
        described(_lib.SSD_F32, (b, H, C, Q)), none, none, described(_lib.SSD_BF16, (b, C, H, P, N)),
        described(_lib.SSD_F32, (b, H, P, N)), small, 1, None)
    assert rc == -2, rc                      # SSD_ERR_SHAPE


def test_static_entry_point_inside_a_hip_graph(oracle):
    # What the entry point is for: a caller that may not allocate, here HIP graph capture.  The call is captured once
    # (its scratch is cleared by a kernel, not by a memset node) and replayed three times, with eager work and
    # synchronisations between the replays and new input values each time; every replay must give the bits of an
    # eager call on the same values.
    import ssd_amd as ops
    d = oracle.make_inputs(2, b=1, L=8192, H=16)
    B, x, dt, dA = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    init = _dev(d["initial_states"])
    b, L, H, P = x.shape
    N, C = B.shape[-1], dt.shape[2]
    out = torch.empty((b, C, H, P, N), device="cuda")
    fin = torch.empty((b, H, P, N), device="cuda")
    x_live = x.clone()
    print(f"[static.graph] x{tuple(x.shape)} chunks={C}", flush=True)
    ops._fused_chunk_state_state_passing_fwd_static(B, x_live, dt, dA, out, fin, initial_states=init)   # set-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops._fused_chunk_state_state_passing_fwd_static(B, x_live, dt, dA, out, fin, initial_states=init)
    for scale in (1.0, -0.5, 3.0):
        x_live.copy_((x.float() * scale).to(x.dtype))
        out.fill_(float("nan")); fin.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert ops._fused_static_status() == 0
        want_out, want_fin = ops._fused_chunk_state_state_passing_fwd(B, x_live, dt, dA, torch.float32, initial_states=init, _kernel=1)
        torch.cuda.synchronize()
        assert torch.equal(out, want_out) and torch.equal(fin, want_fin), f"replay with x * {scale}"
    ref_out, _ = oracle.fused_ref(d["B"], (d["x"].float() * 3.0).to(d["x"].dtype), d["dt"], d["dA_cumsum"],
                                  initial_states=d["initial_states"])
    err = (out.cpu() - ref_out).abs()
    assert int((err > 1e-3 + 2e-3 * ref_out.abs()).sum()) == 0, f"max abs err {float(err.max()):.3e}"
