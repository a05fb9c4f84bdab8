"""GPU parity of the fused call that also computes the scan's state half (ssd_fused_chunk_state_passing_scan_fwd): chunk
state + state passing (kernels/fused_concurrent.py:255-331) and y = scale * C . (state entering the chunk)
(kernels/ssd_chunk_scan.py:94-117) in one launch of the ticket / flag-chain kernel, with and without the passed states
as an output.  Checked against the CPU oracle: chunk_scan_states_ref applied to fused_ref's `out`, rtol 2e-3 /
atol 1e-3 for fp32 y (the state enters the matrix cores as bf16 hi + lo), one bf16 rounding more for bf16 y."""
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-3, 1e-3
LOCAL, GLOBAL = 2, 3


@pytest.fixture(scope="module")
def ops():
    import ssd_amd
    from ssd_amd import _lib
    _lib.load()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return ssd_amd


def _dev(t):
    return None if t is None else t.cuda()


def _mismatches(got, want, rtol=RTOL, atol=ATOL):
    got, want = got.float().cpu(), want.float()
    assert got.shape == want.shape
    assert torch.isfinite(got).all()
    err = (got - want).abs()
    return int((err > atol + rtol * want.abs()).sum()), float(err.max())


def _want(oracle, d, clamp=True):
    out, fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"],
                                seq_idx=d["seq_idx"], clamp=clamp)
    y = oracle.chunk_scan_states_ref(d["C"], out, d["dA_cumsum"], seq_idx=d["seq_idx"])
    return out, fin, y


def _case(ops, oracle, d, name, kernel=1, r=0, with_out=True, y_dtype=torch.float32, accumulate=False, want=None):
    want_out, want_fin, want_y = want if want is not None else _want(oracle, d)
    x = d["x"]
    y0 = None
    if accumulate:
        g = torch.Generator().manual_seed(7)
        y0 = torch.randn(x.shape, generator=g).to(y_dtype)
    from ssd_amd import _lib
    B_ = d["B"]
    dims = _lib.dims_arg(x.shape[0], x.shape[1], x.shape[2], x.shape[3], B_.shape[-1], B_.shape[2], d["dt"].shape[3], d["dt"].shape[2])
    need = int(_lib.load().ssd_fused_scan_workspace_bytes(dims, 1 if with_out else 0, r))
    ws = torch.full((max(need // 4 + 1, 1 << 16),), -1, dtype=torch.int32, device="cuda")    # garbage on purpose, the fp32 slots included
    print(f"[{name}] kernel={kernel} r={r} out={with_out} y={y_dtype} acc={accumulate} x{tuple(x.shape)} seq={d['seq_idx'] is not None}", flush=True)
    y_arg = None if y0 is None else y0.cuda()
    out, fin, y = ops._fused_chunk_state_state_passing_scan_fwd(
        _dev(d["B"]), _dev(x), _dev(d["C"]), _dev(d["dt"]), _dev(d["dA_cumsum"]), torch.float32,
        initial_states=_dev(d["initial_states"]), seq_idx=_dev(d["seq_idx"]), y=y_arg, y_dtype=y_dtype, accumulate=accumulate,
        return_states=with_out, _kernel=kernel, _chunks_per_item=r, _workspace=ws)
    assert ops._fused_workspace_status(ws) == 0
    assert (out is not None) == with_out and y.dtype == y_dtype
    ref_y = want_y if y0 is None else want_y + y0.float()
    extra = 0.0 if y_dtype == torch.float32 else 2.0 ** -8
    checks = [("final", fin, want_fin, RTOL, ATOL), ("y", y, ref_y, RTOL + extra, ATOL + (2.0 ** -8 if accumulate and extra else 0.0))]
    if with_out:
        checks.append(("out", out, want_out, RTOL, ATOL))
    for what, got, wnt, rtol, atol in checks:
        bad, worst = _mismatches(got, wnt, rtol, atol)
        print(f"[{name}.{what}] max_abs={worst:.3e} mismatches={bad}/{wnt.numel()}", flush=True)
        assert bad == 0, f"{name}.{what}: {bad} mismatches, max abs err {worst:.3e}"
    return out, fin, y


SHAPES = [
    dict(b=2, L=2048, H=8, init=True),                   # 8 chunks, initial states
    dict(L=2000, H=8, nseq=5, init=True),                # ragged last chunk, packed sequences (starts inside chunks)
    dict(L=2304, H=8),                                   # 9 chunks: items of 2 or 4 chunks do not divide them
    dict(Q=128, L=1408, N=64, H=8),                      # chunk 128, dstate 64
    dict(P=128, H=4, G=2, L=1280),                       # headdim 128, grouped B and C
    dict(L=257, H=8),                                    # one full chunk and one token
    dict(b=1, L=8192, H=16, nseq=3),                     # 32 chunks on few units: every workgroup waits on the chain
]


@pytest.mark.parametrize("with_out", [True, False], ids=["out", "noout"])
@pytest.mark.parametrize("kernel", [LOCAL, GLOBAL], ids=["local", "global"])
@pytest.mark.parametrize("kw", SHAPES, ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))
def test_fused_scan_variants(ops, oracle, kw, kernel, with_out):
    base = dict(b=2, L=1024, H=6, G=1)
    base.update(kw)
    d = oracle.make_inputs(1, **base)
    want = _want(oracle, d)
    _case(ops, oracle, d, f"scan.k{kernel}", kernel=kernel, with_out=with_out, want=want)


@pytest.mark.parametrize("accumulate", [False, True], ids=["write", "add"])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16], ids=["y32", "y16"])
def test_fused_scan_output_types(ops, oracle, y_dtype, accumulate):
    d = oracle.make_inputs(3, L=4096, H=8, nseq=6, init=True)
    want = _want(oracle, d)
    for with_out in (True, False):
        _case(ops, oracle, d, "scan.types", kernel=1, with_out=with_out, y_dtype=y_dtype, accumulate=accumulate, want=want)


def test_fused_scan_sequence_starts_everywhere(ops, oracle):
    # starts mid-chunk in an item's first chunk (the tokens in front still take the entering state), on a chunk's first
    # token, two in one item, and in an item's last chunk
    d = oracle.make_inputs(1, b=2, L=4096, H=8, init=True)
    starts = [256 + 100, 4 * 256 + 3, 6 * 256, 7 * 256 + 255, 11 * 256 + 17]
    ids = torch.zeros(4096, dtype=torch.int32)
    for s0 in starts:
        ids[s0:] += 1
    d["seq_idx"] = ids.reshape(1, -1).expand(2, -1).contiguous()
    want = _want(oracle, d)
    for kernel in (LOCAL, GLOBAL):
        for with_out in (True, False):
            _case(ops, oracle, d, f"scan.cut.k{kernel}", kernel=kernel, with_out=with_out, want=want)


def test_fused_scan_equals_the_two_calls(ops, oracle):
    # the one-launch result against the library's own fused call followed by its stand-alone consumer
    d = oracle.make_inputs(2, b=2, L=4096, H=16)
    args = [_dev(d[k]) for k in ("B", "x")]
    Cd, dtd, dAd, initd = _dev(d["C"]), _dev(d["dt"]), _dev(d["dA_cumsum"]), _dev(d["initial_states"])
    out2, fin2 = ops._fused_chunk_state_state_passing_fwd(*args, dtd, dAd, torch.float32, initial_states=initd)
    y2 = ops._chunk_scan_states_fwd(Cd, out2, dAd, out_dtype=torch.float32)
    out, fin, y = ops._fused_chunk_state_state_passing_scan_fwd(*args, Cd, dtd, dAd, torch.float32, initial_states=initd,
                                                                y_dtype=torch.float32, _kernel=1)
    torch.cuda.synchronize()
    assert ops.fused_status() == 0
    assert float((out - out2).abs().max()) <= 1e-4 and float((fin - fin2).abs().max()) <= 1e-4
    assert float((y - y2).abs().max()) <= 2e-3
    # left to the library, a call that wants `out` as well IS those two calls (the one-launch kernel saves nothing
    # there): same bits
    out3, fin3, y3 = ops._fused_chunk_state_state_passing_scan_fwd(*args, Cd, dtd, dAd, torch.float32, initial_states=initd,
                                                                   y_dtype=torch.float32)
    torch.cuda.synchronize()
    assert torch.equal(out3, out2) and torch.equal(fin3, fin2) and torch.equal(y3, y2)
    # ... and without `out` it is the one launch
    none, fin4, y4 = ops._fused_chunk_state_state_passing_scan_fwd(*args, Cd, dtd, dAd, torch.float32, initial_states=initd,
                                                                   y_dtype=torch.float32, return_states=False)
    torch.cuda.synchronize()
    assert none is None and ops.fused_status() == 0
    assert float((fin4 - fin2).abs().max()) <= 1e-4 and float((y4 - y2).abs().max()) <= 2e-3


def test_fused_scan_falls_back_where_the_chain_kernel_does_not_apply(ops, oracle):
    # fp32 inputs (the plain kernels): with `out` the call is the two stand-alone calls; without, the wrapper lends a place
    d = oracle.make_inputs(0, L=1024, H=4)
    want_out, want_fin, want_y = _want(oracle, d)
    for with_out in (True, False):
        out, fin, y = ops._fused_chunk_state_state_passing_scan_fwd(
            _dev(d["B"]), _dev(d["x"]), _dev(d["C"]), _dev(d["dt"]), _dev(d["dA_cumsum"]), torch.float32,
            y_dtype=torch.float32, return_states=with_out)
        torch.cuda.synchronize()
        assert (out is not None) == with_out
        assert _mismatches(fin, want_fin)[0] == 0 and _mismatches(y, want_y)[0] == 0


@pytest.mark.timeout(600)
@pytest.mark.parametrize("cfg", [1, 2, 3], ids=["cfg1", "cfg2", "cfg3"])
def test_fused_scan_at_benchmark_configs(ops, oracle, cfg):
    d = oracle.make_inputs(cfg)
    want = _want(oracle, d)
    _case(ops, oracle, d, f"scan.cfg{cfg}", kernel=1, with_out=False, y_dtype=torch.bfloat16, want=want)
    _case(ops, oracle, d, f"scan.cfg{cfg}", kernel=1, with_out=True, y_dtype=torch.float32, want=want)


@pytest.mark.timeout(900)
def test_fused_scan_long_grouped_config_slicewise(ops, oracle):
    # b=1, L=131072, 128 heads in 8 groups, at full size and without the passed states as an output: one head of four
    # different groups against the oracle (its fp32 evaluation of all 128 heads would not fit a few minutes)
    d = oracle.make_inputs(4)
    x, B, C, dt, dAcs = d["x"], d["B"], d["C"], d["dt"], d["dA_cumsum"]
    print(f"[scan.cfg4] x{tuple(x.shape)} B{tuple(B.shape)}", flush=True)
    out, fin, y = ops._fused_chunk_state_state_passing_scan_fwd(_dev(B), _dev(x), _dev(C), _dev(dt), _dev(dAcs), torch.float32,
                                                                y_dtype=torch.bfloat16, return_states=False, _kernel=1)
    torch.cuda.synchronize()
    assert out is None and ops.fused_status() == 0
    ratio = x.shape[2] // B.shape[2]
    for h in (0, 17, 63, 127):
        g = h // ratio
        wo, wf = oracle.fused_ref(B[:, :, g:g + 1], x[:, :, h:h + 1], dt[:, h:h + 1], dAcs[:, h:h + 1])
        wy = oracle.chunk_scan_states_ref(C[:, :, g:g + 1], wo, dAcs[:, h:h + 1])
        for what, got, want, rtol in (("final", fin[:, h:h + 1], wf, RTOL), ("y", y[:, :, h:h + 1], wy, RTOL + 2.0 ** -8)):
            bad, worst = _mismatches(got, want, rtol, ATOL)
            print(f"[scan.cfg4.h{h}.{what}] max_abs={worst:.3e} mismatches={bad}/{want.numel()}", flush=True)
            assert bad == 0, (h, what, bad, worst)
    ops.release_workspaces()
