"""GPU parity on inputs and options the five benchmark configurations do not reach: the fused reference kernels'
un-clamped decay, the reference's own test case, 64-bit seq_idx, dt / dA_cumsum rows that are not contiguous, large
and small magnitudes, a head that does not decay.  Everything goes through the C ABI and is compared with the CPU
oracle.  Tolerance: rtol 2e-3 / atol 1e-3 (fp32 outputs); bf16 outputs at the reference's own self-check tolerance
rtol 1e-2 / atol 1e-3 (main.py:121)."""
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


def _check(name, got, want, rtol=RTOL, atol=ATOL):
    got, want = got.float().cpu(), want.float()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert torch.isfinite(got).all(), name
    err = (got - want).abs()
    nbad = int((err > atol + rtol * want.abs()).sum())
    print(f"[{name}] max_abs={float(err.max()):.3e} max_ref={float(want.abs().max()):.3e} mismatches={nbad}/{want.numel()}",
          flush=True)
    assert nbad == 0, f"{name}: {nbad} mismatches, max abs err {float(err.max()):.3e}"


# kernel families of the fused call: the library's choice, the hook values of ssd_set_token_split, the chain kernel
FAMILIES = [("auto", 0, 0), ("four-tile", 1, 0), ("split2", 2, 0), ("split4", 4, 0), ("chain", 0, 1)]


def _fused(ops, d, split, kernel, out_dtype=torch.float32, clamp=True, states=None, dt=None, dA=None, seq=None):
    old = ops.set_token_split(split)
    try:
        out, fin = ops._fused_chunk_state_state_passing_fwd(
            _dev(d["B"]), _dev(d["x"]), _dev(d["dt"]) if dt is None else dt, _dev(d["dA_cumsum"]) if dA is None else dA,
            out_dtype, initial_states=_dev(d["initial_states"]), seq_idx=_dev(d["seq_idx"]) if seq is None else seq,
            states=states, _clamp=clamp, _kernel=kernel)
        torch.cuda.synchronize()
    finally:
        ops.set_token_split(old)
    return out, fin


@pytest.mark.parametrize("family", FAMILIES, ids=[f[0] for f in FAMILIES])
def test_unclamped_decay_on_every_kernel_family(ops, oracle, family):
    # The reference's fused kernels evaluate exp(dA_last - dA_k) without the min(., 0) of its unfused kernel
    # (fused_globalbar.py:106 against ssd_chunk_state.py:153).  The two agree for a non-increasing dA_cumsum; this one
    # is not, so `clamp` matters, and both settings are checked on every kernel that can serve the call.
    _, split, kernel = family
    d = oracle.make_inputs(1, b=2, L=2048, H=8, init=True)
    g = torch.Generator().manual_seed(11)
    d["dA_cumsum"] = d["dA_cumsum"] + 0.3 * torch.randn(d["dA_cumsum"].shape, generator=g)
    wants = {c: oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"], clamp=c)
             for c in (True, False)}
    assert float((wants[True][0] - wants[False][0]).abs().max()) > 1e-2
    for clamp in (True, False):
        out, fin = _fused(ops, d, split, kernel, clamp=clamp)
        _check(f"{family[0]}.clamp{int(clamp)}.out", out, wants[clamp][0])
        _check(f"{family[0]}.clamp{int(clamp)}.final", fin, wants[clamp][1])
    # ... and the unfused chunk-state call
    for clamp in (True, False):
        old = ops.set_token_split(split)
        try:
            st = ops.ops._chunk_state_impl(_dev(d["B"]), _dev(d["x"]), _dev(d["dt"]), _dev(d["dA_cumsum"]), None, None, True, clamp)
            torch.cuda.synchronize()
        finally:
            ops.set_token_split(old)
        _check(f"{family[0]}.clamp{int(clamp)}.states", st,
               oracle.chunk_state_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], clamp=clamp))


@pytest.mark.parametrize("family", FAMILIES, ids=[f[0] for f in FAMILIES])
def test_reference_own_test_case(ops, oracle, family):
    # kernels/rand_data.py:4-25 as main.py:166-179 runs it: b=1 L=2048 H=80, dt in [0.5, 1) plus a bias in +-0.25,
    # A in (-1, 0] (a head with A = 0 does not decay at all), dt_softplus=False, passed states in C's type (bf16),
    # composed exactly as main.py:63-69 (unfused) and main.py:84-85 / :99-100 (fused).
    _, split, kernel = family
    x, A, B, C, D, dt_raw, dt_bias = oracle.make_reference_inputs()
    Q = 256
    want_dA, want_dt = oracle.chunk_cumsum_ref(dt_raw, A, Q, dt_bias=dt_bias, dt_softplus=False)
    want_states = oracle.chunk_state_ref(B, x, want_dt, want_dA)
    want_out, want_fin = oracle.fused_ref(B, x, want_dt, want_dA)
    xd, Ad, Bd, dtd, biasd = map(_dev, (x, A, B, dt_raw, dt_bias))
    old = ops.set_token_split(split)
    try:
        dA_cumsum, dt = ops._chunk_cumsum_fwd(dtd, Ad, Q, dt_bias=biasd, dt_softplus=False)
        _check("ref.dt", dt, want_dt, 1e-5, 1e-6)
        _check("ref.dA_cumsum", dA_cumsum, want_dA, 1e-4, 1e-5)
        # main.py:64-69
        states = ops._chunk_state_fwd(Bd, xd, dt, dA_cumsum, seq_idx=None, states_in_fp32=True)
        _check("ref.unfused.chunk_state", states, want_states)
        passed, final = ops._state_passing_fwd(states.flatten(-2), dA_cumsum[:, :, :, -1], initial_states=None,
                                               seq_idx=None, chunk_size=Q, out_dtype=C.dtype)
        assert passed.dtype == torch.bfloat16
        _check("ref.unfused.states", passed.reshape(want_out.shape), want_out, 1e-2, 1e-3)
        _check("ref.unfused.final", final.reshape(want_fin.shape), want_fin)
        # main.py:85 / :100 (fp32 as well: the kernel family that serves it differs)
        for name, fn in (("globalbar", ops._fused_chunk_state_state_passing_fwd_globalbar),
                         ("concurrent", ops._fused_chunk_state_state_passing_fwd_concurrent)):
            out, fin = fn(Bd, xd, dt, dA_cumsum, C.dtype, initial_states=None, seq_idx=None, states_in_fp32=True)
            assert out.dtype == torch.bfloat16
            _check(f"ref.{name}.states", out, want_out, 1e-2, 1e-3)
            _check(f"ref.{name}.final", fin, want_fin)
        out, fin = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dt, dA_cumsum, torch.float32, _kernel=kernel)
        _check("ref.fused.fp32.states", out, want_out)
        _check("ref.fused.fp32.final", fin, want_fin)
    finally:
        ops.set_token_split(old)


def test_int64_seq_idx(ops, oracle):
    # the reference does not assert the type of seq_idx; upstream passes int32, torch defaults to int64
    d = oracle.make_inputs(3, L=4096, H=8, nseq=5)
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], seq_idx=d["seq_idx"])
    seq64 = _dev(d["seq_idx"]).to(torch.int64)
    for name, split, kernel in FAMILIES:
        out, fin = _fused(ops, d, split, kernel, seq=seq64)
        _check(f"seq64.{name}.out", out, want_out)
        _check(f"seq64.{name}.final", fin, want_fin)
    st = ops._chunk_state_fwd(_dev(d["B"]), _dev(d["x"]), _dev(d["dt"]), _dev(d["dA_cumsum"]), seq_idx=seq64)
    _check("seq64.states", st, oracle.chunk_state_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], seq_idx=d["seq_idx"]))
    o2, f2 = ops._state_passing_fwd(st.flatten(-2), _dev(d["dA_cumsum"])[:, :, :, -1], seq_idx=seq64, chunk_size=256)
    _check("seq64.state_passing", o2.reshape(want_out.shape), want_out)


def test_dt_rows_with_a_stride(ops, oracle):
    # dt and dA_cumsum as every second element of a wider buffer: the kernels that fetch 16 bytes of them at a time do
    # not apply, the call must still be served
    d = oracle.make_inputs(1, b=2, L=1024, H=8, init=True)
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
    want_states = oracle.chunk_state_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"])

    def strided(t):
        wide = torch.full(t.shape[:-1] + (2 * t.shape[-1],), float("nan"), device="cuda")
        wide[..., ::2] = _dev(t)
        v = wide[..., ::2]
        assert v.stride(-1) == 2
        return v

    dt_s, dA_s = strided(d["dt"]), strided(d["dA_cumsum"])
    for name, split, kernel in FAMILIES[:4]:
        out, fin = _fused(ops, d, split, 0, dt=dt_s, dA=dA_s)
        _check(f"strided.{name}.out", out, want_out)
        _check(f"strided.{name}.final", fin, want_fin)
    st = ops._chunk_state_fwd(_dev(d["B"]), _dev(d["x"]), dt_s, dA_s)
    _check("strided.states", st, want_states)


@pytest.mark.parametrize("scale", [2.0 ** 10, 2.0 ** -10], ids=["x1024", "x1over1024"])
@pytest.mark.parametrize("family", FAMILIES, ids=[f[0] for f in FAMILIES])
def test_magnitudes(ops, oracle, family, scale):
    # x and B both scaled by 2^10 or 2^-10 (exact in bf16): the states scale by 2^20 / 2^-20.  The bf16 hi + lo split of
    # x * w keeps its relative accuracy; the comparison is made on the states scaled back.
    _, split, kernel = family
    d = oracle.make_inputs(1, b=2, L=1024, H=8, init=False)
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"])
    d2 = dict(d)
    d2["x"] = (d["x"].float() * scale).to(d["x"].dtype)
    d2["B"] = (d["B"].float() * scale).to(d["B"].dtype)
    out, fin = _fused(ops, d2, split, kernel)
    _check(f"scale.{family[0]}.out", out / scale ** 2, want_out)
    _check(f"scale.{family[0]}.final", fin / scale ** 2, want_fin)


@pytest.mark.parametrize("family", FAMILIES, ids=[f[0] for f in FAMILIES])
def test_head_without_decay(ops, oracle, family):
    # A = 0 for some heads: dA_cumsum is zero, every weight is dt, the state is a plain running sum that grows with L
    _, split, kernel = family
    d = oracle.make_inputs(1, b=1, L=4096, H=8, init=True)
    A = d["A"].clone()
    A[::3] = 0.0
    d["dA_cumsum"], d["dt"] = oracle.chunk_cumsum_ref(d["dt_raw"], A, 256, dt_bias=d["dt_bias"], dt_softplus=True)
    assert float(d["dA_cumsum"][:, 0].abs().max()) == 0.0
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
    out, fin = _fused(ops, d, split, kernel)
    _check(f"nodecay.{family[0]}.out", out, want_out)
    _check(f"nodecay.{family[0]}.final", fin, want_fin)
