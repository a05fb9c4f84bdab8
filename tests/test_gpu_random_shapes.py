"""Seeded random shapes through the fused call (the library's own kernel choice, then the chain kernel insisted on with
a random number of chunks per item and either way of crossing compute units) against the CPU oracle on the same
inputs.  The hand-picked cases of the other files name their corner; these draw combinations nobody thought of: ragged
last chunks, sequence starts anywhere, chunk counts that items do not divide, one to eight groups, with and without
initial states.  Reference semantics: kernels/fused_globalbar.py:201-266; tolerance rtol 2e-3 / atol 1e-3 (bf16 inputs,
fp32 states)."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-3, 1e-3


@pytest.fixture(scope="module")
def ops():
    import ssd_amd
    from ssd_amd import _lib
    _lib.load()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return ssd_amd


def _dev(t):
    return None if t is None else t.cuda()


def _draw(seed):
    rng = random.Random(9000 + seed)
    P = rng.choice([32, 64, 64, 128])
    G = rng.choice([1, 1, 2, 4])
    per_group = rng.choice([1, 2, 3]) * (128 // P)            # heads per group: four 32-row tiles per (batch, group) or a multiple
    kw = dict(b=rng.choice([1, 1, 2, 3]), H=G * per_group, P=P, G=G, N=rng.choice([64, 128, 128]), Q=rng.choice([128, 256, 256]),
              init=rng.random() < 0.5)
    kw["L"] = rng.randrange(kw["Q"] + 1, 12 * kw["Q"])        # 2 .. 12 chunks, mostly with a ragged last one
    if rng.random() < 0.5:
        kw["nseq"] = rng.randrange(2, 7)
    return kw, rng.choice([2, 3]), rng.choice([1, 2, 4])


@pytest.mark.parametrize("seed", range(24))
def test_random_shape(ops, oracle, seed):
    kw, kernel, r = _draw(seed)
    d = oracle.make_inputs(2 if "nseq" not in kw else 3, **kw)
    x, B, dt, dA, seq, init = d["x"], d["B"], d["dt"], d["dA_cumsum"], d["seq_idx"], d["initial_states"]
    want_out, want_fin = oracle.fused_ref(B, x, dt, dA, initial_states=init, seq_idx=seq)
    args = [_dev(t) for t in (B, x, dt, dA)]
    for name, extra in (("auto", {}), (f"chain{kernel}x{r}", dict(_kernel=kernel, _chunks_per_item=r))):
        ws = torch.full((1 << 16,), -1, dtype=torch.int32, device="cuda")
        print(f"[random {seed}] {kw} {name}", flush=True)
        out, fin = ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, initial_states=_dev(init), seq_idx=_dev(seq),
                                                            _workspace=ws, **extra)
        torch.cuda.synchronize()
        assert ops._fused_workspace_status(ws) == 0
        for what, got, want in (("out", out, want_out), ("final", fin, want_fin)):
            got = got.float().cpu()
            assert torch.isfinite(got).all(), (seed, name, what)
            err = (got - want).abs()
            bad = int((err > ATOL + RTOL * want.abs()).sum())
            assert bad == 0, f"seed {seed} {kw} {name}.{what}: {bad} mismatches, max abs err {float(err.max()):.3e}"
    # the forced chain launch again with bf16 passed states, on the wrapper's own workspace: the running state crosses
    # between work items in fp32, so the final states are the same bits and `out` is the fp32 `out` rounded once (the
    # number of chunks per item does not change the arithmetic; with bf16 `out` it is at least two)
    out16, fin16 = ops._fused_chunk_state_state_passing_fwd(*args, torch.bfloat16, initial_states=_dev(init), seq_idx=_dev(seq),
                                                            _kernel=kernel, _chunks_per_item=max(r, 2))
    torch.cuda.synchronize()
    assert torch.equal(fin16, fin), f"seed {seed} {kw}: final states with bf16 out differ, max {float((fin16 - fin).abs().max()):.3e}"
    assert torch.equal(out16, out.to(torch.bfloat16)), f"seed {seed} {kw}: bf16 out is not the fp32 out rounded"


def _draw_any(seed):
    """Anything the entry points accept: element types, sizes off every tiling, strided chunk-end decay."""
    rng = random.Random(7000 + seed)
    G = rng.choice([1, 1, 2, 3])
    kw = dict(b=rng.choice([1, 2, 3]), H=G * rng.choice([1, 2, 4, 5]), G=G, P=rng.choice([16, 32, 40, 64, 128]),
              N=rng.choice([16, 24, 64, 128]), Q=rng.choice([64, 128, 256]), init=rng.random() < 0.5,
              dtype=rng.choice(["bf16", "bf16", "fp32", "fp16"]))
    kw["L"] = rng.randrange(kw["Q"] // 2, 6 * kw["Q"])         # 1 .. 6 chunks, the single one possibly short
    if rng.random() < 0.4 and kw["L"] > 600:
        kw["nseq"] = rng.randrange(2, 5)
    return kw, rng.choice([torch.float32, torch.float32, torch.bfloat16]), rng.random() < 0.5


@pytest.mark.parametrize("seed", range(24))
def test_random_arguments_without_a_workspace(ops, oracle, seed):
    # the three entry points of the path on whatever the draw gives: fused (with and without a `states` output, fp32 or
    # bf16 passed states), chunk state, state passing -- every kernel family is somebody's fallback here
    kw, out_dtype, with_states = _draw_any(seed)
    d = oracle.make_inputs(3 if "nseq" in kw else 1, **kw)
    x, B, dt, dA, seq, init = d["x"], d["B"], d["dt"], d["dA_cumsum"], d["seq_idx"], d["initial_states"]
    print(f"[random-any {seed}] {kw} out {out_dtype} states {with_states}", flush=True)
    want_states = oracle.chunk_state_ref(B, x, dt, dA, seq_idx=seq)
    want_out, want_fin = oracle.fused_ref(B, x, dt, dA, initial_states=init, seq_idx=seq)
    xd, Bd, dtd, dAd, seqd, initd = map(_dev, (x, B, dt, dA, seq, init))
    b, L, H, P = x.shape
    N, C = B.shape[-1], dt.shape[2]

    def check(what, got, want, rtol=RTOL, atol=ATOL):
        got = got.float().cpu()
        assert got.shape == want.shape and torch.isfinite(got).all(), (seed, what)
        err = (got - want.float()).abs()
        bad = int((err > atol + rtol * want.abs()).sum())
        assert bad == 0, f"seed {seed} {kw} {what}: {bad} mismatches, max abs err {float(err.max()):.3e}"

    st_buf = torch.full((b, C, H, P, N), float("nan"), device="cuda") if with_states else None
    out, fin = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, out_dtype, initial_states=initd, seq_idx=seqd,
                                                        states=st_buf)
    torch.cuda.synchronize()
    check("out", out, want_out, *((1e-2, 1e-3) if out_dtype != torch.float32 else (RTOL, ATOL)))
    check("final", fin, want_fin)
    if with_states:
        check("states", st_buf, want_states)
    st = ops._chunk_state_fwd(Bd, xd, dtd, dAd, seq_idx=seqd)
    check("chunk_state", st, want_states)
    o2, f2 = ops._state_passing_fwd(st.flatten(-2), dAd[:, :, :, -1], initial_states=None if initd is None else initd.flatten(-2),
                                    seq_idx=seqd, chunk_size=dt.shape[-1])
    torch.cuda.synchronize()
    check("state_passing.out", o2.reshape(b, C, H, P, N), want_out)
    check("state_passing.final", f2.reshape(b, H, P, N), want_fin)


@pytest.mark.parametrize("seed", range(16))
def test_random_neighbours_of_the_path(ops, oracle, seed):
    # the producer of dt / dA_cumsum (kernels/ssd_chunk_state.py:33-79) and the consumer of the passed states
    # (kernels/ssd_chunk_scan.py:94-117) on drawn sizes and element types, both matrix-core scan kernels in turn
    kw, _, _ = _draw_any(seed + 100)
    d = oracle.make_inputs(3 if "nseq" in kw else 1, **kw)
    Q = d["cfg"]["Q"]
    rng = random.Random(seed)
    softplus, use_bias = rng.random() < 0.6, rng.random() < 0.6
    limit = rng.choice([(0.0, float("inf")), (2e-3, 5e-2)])
    raw, A, bias = d["dt_raw"], d["A"], d["dt_bias"] if use_bias else None
    print(f"[random-neighbours {seed}] {kw} softplus {softplus} bias {use_bias} limit {limit}", flush=True)
    want_da, want_dt = oracle.chunk_cumsum_ref(raw, A, Q, dt_bias=bias, dt_softplus=softplus, dt_limit=limit)
    got_da, got_dt = ops._chunk_cumsum_fwd(_dev(raw), _dev(A), Q, dt_bias=_dev(bias), dt_softplus=softplus, dt_limit=limit)
    torch.cuda.synchronize()

    def check(what, got, want, rtol, atol):
        got = got.float().cpu()
        assert got.shape == want.shape and torch.isfinite(got).all(), (seed, what)
        err = (got - want.float()).abs()
        bad = int((err > atol + rtol * want.abs()).sum())
        assert bad == 0, f"seed {seed} {kw} {what}: {bad} mismatches, max abs err {float(err.max()):.3e}"

    check("cumsum.dt", got_dt, want_dt, 2e-6, 1e-9)
    check("cumsum.dA_cumsum", got_da, want_da, 1e-5, 1e-6)
    seq, dA = d["seq_idx"], d["dA_cumsum"]
    prev, _ = oracle.fused_ref(d["B"], d["x"], d["dt"], dA, initial_states=d["initial_states"], seq_idx=seq)
    want_y = oracle.chunk_scan_states_ref(d["C"], prev, dA, seq_idx=seq)
    for kernel in (1, 2):
        old = ops.set_scan_kernel(kernel)
        try:
            y = ops._chunk_scan_states_fwd(_dev(d["C"]), _dev(prev), _dev(dA), seq_idx=_dev(seq), out_dtype=torch.float32)
            torch.cuda.synchronize()
        finally:
            ops.set_scan_kernel(old)
        check(f"scan_states[{kernel}]", y, want_y, RTOL, ATOL)
