"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Tolerance (from the benchmark contract): rtol 2e-3 / atol 1e-3 against an fp32 evaluation, bf16 inputs,
fp32 states.  bf16 outputs (out_dtype / states_in_fp32=False) are compared at the reference's own
self-check tolerance rtol 1e-2 / atol 1e-3 (main.py:121)."""
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
    got = got.float().cpu()
    want = want.float()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    err = (got - want).abs()
    bad = err > (atol + rtol * want.abs())
    nbad = int(bad.sum())
    print(f"[{name}] max_abs={float(err.max()):.3e} max_ref={float(want.abs().max()):.3e} mismatches={nbad}/{want.numel()}",
          flush=True)
    assert torch.isfinite(got).all(), name
    assert nbad == 0, f"{name}: {nbad} mismatches, max abs err {float(err.max()):.3e}"


def _run_case(ops, oracle, d, with_states=True, out_dtype=torch.float32, check_unfused=True, name="case"):
    x, B, dt, dAcs = d["x"], d["B"], d["dt"], d["dA_cumsum"]
    seq, init = d["seq_idx"], d["initial_states"]
    print(f"[{name}] x{tuple(x.shape)} {x.dtype} B{tuple(B.shape)} seq={seq is not None} init={init is not None}", flush=True)
    want_states = oracle.chunk_state_ref(B, x, dt, dAcs, seq_idx=seq)
    want_out, want_fin = oracle.fused_ref(B, x, dt, dAcs, initial_states=init, seq_idx=seq)
    xd, Bd, dtd, dAd, seqd, initd = map(_dev, (x, B, dt, dAcs, seq, init))
    b, L, H, P = x.shape
    N = B.shape[-1]
    C = dt.shape[2]
    # poison the outputs: every element must be written by the kernel
    st_buf = torch.full((b, C, H, P, N), float("nan"), device="cuda") if with_states else None
    out, fin = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, out_dtype, initial_states=initd,
                                                        seq_idx=seqd, states=st_buf)
    torch.cuda.synchronize()
    assert out.dtype == out_dtype and fin.dtype == torch.float32
    assert out.shape == (b, C, H, P, N) and fin.shape == (b, H, P, N)
    lo = out_dtype != torch.float32
    _check(name + ".out", out, want_out, *((1e-2, 1e-3) if lo else (RTOL, ATOL)))
    _check(name + ".final", fin, want_fin)
    if with_states:
        _check(name + ".states", st_buf, want_states)
    if check_unfused:
        st = ops._chunk_state_fwd(Bd, xd, dtd, dAd, seq_idx=seqd)
        _check(name + ".chunk_state", st, want_states)
        o2, f2 = ops._state_passing_fwd(st.flatten(-2), dAd[:, :, :, -1],
                                        initial_states=None if initd is None else initd.flatten(-2),
                                        seq_idx=seqd, chunk_size=dt.shape[-1])
        torch.cuda.synchronize()
        _check(name + ".state_passing.out", o2.reshape(b, C, H, P, N), want_out)
        _check(name + ".state_passing.final", f2.reshape(b, H, P, N), want_fin)
        if with_states and not lo:
            # the fused kernel and the unfused chunk-state kernel share the contraction code: with the same token
            # split the states are bit-identical; left to itself the library may pick different splits for the
            # two launches (they differ in the number of independent work items), which only reorders the sum
            forced = ops.set_token_split(0)
            ops.set_token_split(forced)
            if forced in (2, 4):
                assert torch.equal(st, st_buf)
            else:
                assert float((st - st_buf).abs().max()) <= 1e-4
    return out, fin


# ------------------------------------------------------------------ the five benchmark configurations
def test_config0_fp32_generic_path(ops, oracle):
    _run_case(ops, oracle, oracle.make_inputs(0), name="cfg0")


@pytest.mark.parametrize("kw", [
    dict(),                                              # the configuration itself: fp32 inputs
    dict(L=1000, nseq=3, init=True),                     # ragged last chunk, packed sequences, initial states
    dict(L=300, H=3, P=40, N=24, Q=64, dtype="bf16"),    # bf16, but sizes only the plain kernel takes
    dict(L=256),                                         # one chunk: nothing to split
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()) or "cfg0")
def test_plain_kernel_fused_call_as_chunk_states_plus_recurrence(ops, oracle, kw):
    # arguments only the plain FMA kernel takes: with two chunks or more the fused call runs as that kernel's chunk-state
    # launch into `out` (or `states=`) + the recurrence in place; a forced kernel family keeps it on the fused launch.
    # Both against the oracle (fused_globalbar.py:201-266 semantics) and against each other.
    d = oracle.make_inputs(0, **kw)
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    init, seq = _dev(d["initial_states"]), _dev(d["seq_idx"])
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"],
                                          seq_idx=d["seq_idx"])
    want_states = oracle.chunk_state_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], seq_idx=d["seq_idx"])
    results = []
    for forced in (0, 2):
        old = ops.set_token_split(forced)
        try:
            out, fin = ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, initial_states=init, seq_idx=seq)
            states = torch.full(want_states.shape, float("nan"), device="cuda")
            out_s, fin_s = ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, initial_states=init, seq_idx=seq,
                                                                    states=states)
            torch.cuda.synchronize()
        finally:
            ops.set_token_split(old)
        for what, got, want in (("out", out, want_out), ("final", fin, want_fin), ("out+states", out_s, want_out),
                                ("final+states", fin_s, want_fin), ("states", states, want_states)):
            _check(f"plain[{forced}].{what}", got, want)
        results.append((out, fin))
    assert float((results[0][0] - results[1][0]).abs().max()) <= 1e-4
    assert float((results[0][1] - results[1][1]).abs().max()) <= 1e-4


def test_config1_mamba2_130m(ops, oracle):
    _run_case(ops, oracle, oracle.make_inputs(1), name="cfg1")


@pytest.mark.timeout(600)
def test_config2_mamba2_2p7b_with_initial_states(ops, oracle):
    _run_case(ops, oracle, oracle.make_inputs(2), name="cfg2")


@pytest.mark.timeout(600)
def test_config3_varlen_packed(ops, oracle):
    d = oracle.make_inputs(3)
    out, fin = _run_case(ops, oracle, d, name="cfg3")
    # packed == solo: the final state is the last sequence evaluated alone from a zero state
    n_last = int(d["seq_lens"][-1])
    sl = slice(d["x"].shape[1] - n_last, None)
    hs = [0, 41, 79]
    o64, f64 = oracle.token_recurrence_ref(d["x"][:, sl][:, :, hs], d["B"][:, sl], d["dt_tok"][:, sl][:, :, hs],
                                           d["A"][hs], 10 ** 9)
    _check("cfg3.final_vs_solo_token_recurrence", fin[:, hs], f64)


@pytest.mark.timeout(900)
def test_config4_long_grouped_slicewise(ops, oracle):
    d = oracle.make_inputs(4)
    x, B, dt, dAcs = d["x"], d["B"], d["dt"], d["dA_cumsum"]
    print(f"[cfg4] x{tuple(x.shape)} B{tuple(B.shape)}", flush=True)
    xd, Bd, dtd, dAd = map(_dev, (x, B, dt, dAcs))
    out, fin = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, torch.float32)
    torch.cuda.synchronize()
    ratio = x.shape[2] // B.shape[2]
    for h in (0, 17, 63, 127):                 # one head of four different groups, compared against the oracle
        g = h // ratio
        wo, wf = oracle.fused_ref(B[:, :, g:g + 1], x[:, :, h:h + 1], dt[:, h:h + 1], dAcs[:, h:h + 1])
        _check(f"cfg4.h{h}.out", out[:, :, h:h + 1], wo)
        _check(f"cfg4.h{h}.final", fin[:, h:h + 1], wf)
    # full-size property: with one token split for both, fused == the library's own unfused kernels, bit for bit and
    # for every head; and the split the library picks by itself agrees with that to rounding
    for waves in (4, 2):
        old = ops.set_token_split(waves)
        try:
            o1, f1 = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, torch.float32)
            st = ops._chunk_state_fwd(Bd, xd, dtd, dAd)
            o2, f2 = ops._state_passing_fwd(st.flatten(-2), dAd[:, :, :, -1])
            torch.cuda.synchronize()
        finally:
            ops.set_token_split(old)
        assert torch.equal(f2.reshape(f1.shape), f1), waves
        assert torch.equal(o2.reshape(o1.shape), o1), waves
        err = max(float((o1 - out).abs().max()), float((f1 - fin).abs().max()))
        print(f"[cfg4.split{waves}_vs_default] max_abs={err:.3e}", flush=True)
        assert err <= 1e-4
        del o1, f1, st, o2, f2


# ------------------------------------------------------------------ shapes, layouts and options beyond the five
@pytest.mark.parametrize("kw", [
    dict(L=1000),                                        # ragged last chunk
    dict(L=1000, nseq=5),                                # ragged + packed sequences
    dict(Q=128, L=1024),                                 # chunk 128
    dict(N=64),                                          # dstate 64 on the bf16 MFMA path
    dict(P=128, H=4),                                    # headdim 128
    dict(H=8, G=4),                                      # grouped B
    dict(L=300, H=3, P=40, N=24, G=1, Q=64),             # nothing aligned: generic path
    dict(dtype="fp16"),                                  # fp16 inputs: generic path
    dict(b=3, L=256, H=5),                               # a single chunk
    dict(L=1),                                           # a single token
    dict(L=33, nseq=2),                                  # one ragged chunk holding two sequences
    dict(L=257, H=8),                                    # one full chunk and one token (four-tile kernel when forced)
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))
def test_small_variants(ops, oracle, kw):
    base = dict(b=2, L=1024, H=6, G=1, init=True)
    base.update(kw)
    _run_case(ops, oracle, oracle.make_inputs(1, **base), name="variant")


@pytest.mark.parametrize("waves", [1, 2, 4])
@pytest.mark.parametrize("kw", [
    dict(),                                              # chunk 256, dstate 128
    dict(L=1000, nseq=5),                                # ragged + packed sequences
    dict(Q=128, L=1024),                                 # chunk 128
    dict(N=64),                                          # dstate 64
    dict(P=128, H=4, G=2),                               # headdim 128, grouped B
    dict(L=1),                                           # a single token
    dict(L=257),                                         # one full chunk and one token
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()) or "base")
def test_token_split_variants(ops, oracle, kw, waves):
    # the bf16 MFMA kernel families behind the hook (the library picks one from the problem size by itself): one
    # wave per tile with four tiles per workgroup (1), two or four waves per tile (2, 4).  The ticket / flag-chain
    # kernel has its own tests (test_gpu_chain.py).
    base = dict(b=2, L=1024, H=6, G=1, init=True)
    base.update(kw)
    old = ops.set_token_split(waves)
    try:
        _run_case(ops, oracle, oracle.make_inputs(1, **base), name=f"split{waves}")
        _run_case(ops, oracle, oracle.make_inputs(1, **base), with_states=False, out_dtype=torch.bfloat16,
                  check_unfused=False, name=f"split{waves}.bf16out")
    finally:
        ops.set_token_split(old)


@pytest.mark.parametrize("chunks", [0, 1, 3, 64])
@pytest.mark.parametrize("kw", [
    dict(L=2304),                                        # 9 chunks: segments of 3 divide them, 1 and 64 do not matter
    dict(L=2000, nseq=5),                                # ragged last chunk + packed sequences
    dict(Q=128, L=1408, N=64),                           # 11 chunks of 128, dstate 64
    dict(P=128, H=4, G=2, L=1280),                       # headdim 128, grouped B, 5 chunks
    dict(L=1),                                           # a single token
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))
def test_chunk_state_segments(ops, oracle, kw, chunks):
    # _chunk_state_fwd on the kernel with four tiles per workgroup: any cut of the chunks into segments gives the
    # same bits, for fp32 and 16-bit states, into a strided view as well
    base = dict(b=2, L=1024, H=6, G=1)
    base.update(kw)
    d = oracle.make_inputs(1, **base)
    x, B, dt, dA, seq = map(_dev, (d["x"], d["B"], d["dt"], d["dA_cumsum"], d["seq_idx"]))
    want = oracle.chunk_state_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], seq_idx=d["seq_idx"])
    old_split, old_chunks = ops.set_token_split(1), ops.set_segment_chunks(chunks)
    try:
        print(f"[segments] x{tuple(x.shape)} chunks/workgroup={chunks}", flush=True)
        st = ops._chunk_state_fwd(B, x, dt, dA, seq_idx=seq)
        _check("segments.fp32", st, want)
        lo = ops._chunk_state_fwd(B, x, dt, dA, seq_idx=seq, states_in_fp32=False)
        assert lo.dtype == x.dtype
        _check("segments.bf16", lo, want, 1e-2, 1e-3)
        b, C, H, P, N = want.shape
        wide = torch.full((b, C, H, P, 2 * N), float("nan"), device="cuda")
        ops._chunk_state_fwd(B, x, dt, dA, seq_idx=seq, states=wide[..., N:])
        assert torch.equal(wide[..., N:], st) and torch.isnan(wide[..., :N]).all()
        ops.set_segment_chunks(2)
        assert torch.equal(ops._chunk_state_fwd(B, x, dt, dA, seq_idx=seq), st)
    finally:
        ops.set_token_split(old_split)
        ops.set_segment_chunks(old_chunks)


@pytest.mark.parametrize("kw", [
    dict(L=65536, Q=128),                                # 16 tiles x 512 chunks
    dict(L=70000, nseq=9, H=16, G=2),                    # ragged, packed sequences, grouped B: 32 tiles x 274 chunks
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))
def test_fused_few_tiles_many_chunks(ops, oracle, kw):
    # fewer than 512 state tiles, at least 8192 tile-chunks, fp32 out, no states= buffer: the fused call runs as the
    # chunk-state launch into `out` and the recurrence in place; with bf16 out it stays on the token-split kernel
    base = dict(b=1, L=1024, H=8, G=1, init=True)
    base.update(kw)
    d = oracle.make_inputs(1, **base)
    _run_case(ops, oracle, d, with_states=False, check_unfused=False, name="in-place")
    _run_case(ops, oracle, d, with_states=False, out_dtype=torch.bfloat16, check_unfused=False, name="in-place.bf16out")
    _run_case(ops, oracle, d, with_states=True, check_unfused=False, name="with-states")


@pytest.mark.parametrize("seed", range(10))
def test_random_shapes_through_the_dispatcher(ops, oracle, seed):
    # seeded random draws over shapes and options, each run with the library choosing the kernels by itself and with
    # the four-tile kernel forced: whatever path the dispatcher takes, the results are the oracle's
    import random
    rng = random.Random(1000 + seed)
    P = rng.choice([32, 64, 128])
    G = rng.choice([1, 2])
    H = G * rng.choice([2, 4, 6])
    Q = rng.choice([128, 256])
    kw = dict(b=rng.choice([1, 2, 3]), H=H, G=G, P=P, N=rng.choice([64, 128]), Q=Q,
              L=rng.choice([Q, 3 * Q + 17, 5 * Q, 9 * Q - 1]), nseq=rng.choice([0, 0, 3]), init=rng.random() < 0.5)
    d = oracle.make_inputs(1, **kw)
    with_states = rng.random() < 0.5
    lowp = rng.random() < 0.3
    for forced in (0, 1):
        old = ops.set_token_split(forced)
        try:
            _run_case(ops, oracle, d, with_states=with_states and not lowp, out_dtype=torch.bfloat16 if lowp else torch.float32,
                      check_unfused=not lowp, name=f"random{seed}.split{forced}")
        finally:
            ops.set_token_split(old)


def test_bf16_outputs(ops, oracle):
    d = oracle.make_inputs(1, b=2, L=1024, H=6, init=True)
    _run_case(ops, oracle, d, with_states=False, out_dtype=torch.bfloat16, check_unfused=False, name="bf16out")
    xd, Bd, dtd, dAd = map(_dev, (d["x"], d["B"], d["dt"], d["dA_cumsum"]))
    st = ops._chunk_state_fwd(Bd, xd, dtd, dAd, states_in_fp32=False)
    assert st.dtype == torch.bfloat16
    _check("bf16 states", st, oracle.chunk_state_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"]), 1e-2, 1e-3)
    o, f = ops._state_passing_fwd(st.flatten(-2), dAd[..., -1], out_dtype=torch.bfloat16)
    wo, wf = oracle.state_passing_ref(st.cpu().flatten(-2), d["dA_cumsum"][..., -1], out_dtype=torch.bfloat16)
    _check("bf16 state passing out", o, wo, 1e-2, 1e-3)
    _check("bf16 state passing final", f, wf)


def test_strided_views_of_a_packed_projection(ops, oracle):
    # x and B carved out of one (b, L, d_inner + 2*G*N) buffer, as a Mamba2 block does: row stride != H*P
    d = oracle.make_inputs(1, b=2, L=512, H=6)
    b, L, H, P = d["x"].shape
    G, N = d["B"].shape[2:]
    packed = torch.zeros(b, L, H * P + 2 * G * N, dtype=torch.bfloat16, device="cuda")
    packed[..., :H * P] = d["x"].cuda().reshape(b, L, H * P)
    packed[..., H * P:H * P + G * N] = d["B"].cuda().reshape(b, L, G * N)
    xv = packed[..., :H * P].view(b, L, H, P)
    Bv = packed[..., H * P:H * P + G * N].view(b, L, G, N)
    assert not xv.is_contiguous()
    out, fin = ops._fused_chunk_state_state_passing_fwd(Bv, xv, d["dt"].cuda(), d["dA_cumsum"].cuda(), torch.float32)
    wo, wf = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"])
    _check("strided.out", out, wo)
    _check("strided.final", fin, wf)


def test_back_to_back_launches_are_deterministic(ops, oracle):
    d = oracle.make_inputs(3, L=8192, H=16, nseq=6)
    args = list(map(_dev, (d["B"], d["x"], d["dt"], d["dA_cumsum"])))
    seq = d["seq_idx"].cuda()
    outs = [ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, seq_idx=seq) for _ in range(4)]
    torch.cuda.synchronize()
    for o, f in outs[1:]:
        assert torch.equal(o, outs[0][0]) and torch.equal(f, outs[0][1])


def test_linearity_at_full_size(ops, oracle):
    """Size-independent property at the benchmark shape: scaling x by 2 scales every output by exactly 2, bit for bit.

    This is also the regression guard of the store-data hazard in the kernels' 16-byte state stores: the data
    registers of a wide store are read out over several cycles after issue, and a following instruction that rewrites
    them (the decay multiplication of the accumulators, the next block's layout change) must be kept away -- the
    `s_nop` behind every such store does that.  Without it a small fraction of the stored values were wrong at this
    size only, and only this bit-exact comparison showed it (the tolerance tests did not).  Both kernel families that
    store whole state tiles are run: the library's choice (the ticket / flag-chain kernel here) and the four-tile
    kernel.  If a compiler update ever schedules around the wait states, this test is what fails: keep it."""
    d = oracle.make_inputs(2)
    Bd, xd, dtd, dAd = map(_dev, (d["B"], d["x"], d["dt"], d["dA_cumsum"]))
    for split in (0, 1):
        old = ops.set_token_split(split)
        try:
            o1, f1 = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, torch.float32)
            o2, f2 = ops._fused_chunk_state_state_passing_fwd(Bd, xd * 2, dtd, dAd, torch.float32)
            torch.cuda.synchronize()
        finally:
            ops.set_token_split(old)
        assert torch.equal(o2, 2 * o1) and torch.equal(f2, 2 * f1), f"token split {split}"
        assert (o1[:, 0] == 0).all()
        del o1, f1, o2, f2


def test_non_default_stream(ops, oracle):
    d = oracle.make_inputs(1, b=1, L=512, H=4)
    Bd, xd, dtd, dAd = map(_dev, (d["B"], d["x"], d["dt"], d["dA_cumsum"]))
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        out, fin = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, torch.float32)
    s.synchronize()
    wo, wf = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"])
    _check("stream.out", out, wo)


def test_reference_module_names_resolve(ops):
    from kernels.ssd_chunk_state import _chunk_state_fwd
    from kernels.ssd_state_passing import _state_passing_fwd
    from kernels.fused_globalbar import _fused_chunk_state_state_passing_fwd_globalbar
    from kernels.fused_concurrent import _fused_chunk_state_state_passing_fwd_concurrent
    assert _chunk_state_fwd is ops._chunk_state_fwd and _state_passing_fwd is ops._state_passing_fwd
    assert callable(_fused_chunk_state_state_passing_fwd_globalbar) and callable(_fused_chunk_state_state_passing_fwd_concurrent)


# ------------------------------------------------------------------ dt preparation + per-chunk cumulative sum
@pytest.mark.parametrize("kw", [
    dict(),                                              # cfg 1 shape: bf16 dt, bias, softplus
    dict(L=1000),                                        # ragged last chunk
    dict(H=5, Q=64, L=512),                              # head count below one tile, chunk 64
    dict(H=40, Q=128),                                   # two head tiles, the second partial
    dict(Q=1024, L=4096, b=1),                           # the largest chunk the kernel takes (> 64 KB of LDS)
    dict(dtype="fp32", b=1, L=1024),                     # fp32 dt
    dict(dtype="fp16", b=1, L=512, H=8),                 # fp16 dt, half a head tile
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()) or "base")
def test_chunk_cumsum(ops, oracle, kw):
    base = dict(b=2, L=2048, H=24)
    base.update(kw)
    d = oracle.make_inputs(1, **base)
    Q = d["cfg"]["Q"]
    raw, A, bias = d["dt_raw"], d["A"], d["dt_bias"]
    for softplus, use_bias, limit in ((True, True, (0.0, float("inf"))), (False, False, (0.0, float("inf"))),
                                      (True, True, (2e-3, 5e-2))):
        want_da, want_dt = oracle.chunk_cumsum_ref(raw, A, Q, dt_bias=bias if use_bias else None, dt_softplus=softplus,
                                                   dt_limit=limit)
        got_da, got_dt = ops._chunk_cumsum_fwd(_dev(raw), _dev(A), Q, dt_bias=_dev(bias) if use_bias else None,
                                               dt_softplus=softplus, dt_limit=limit)
        torch.cuda.synchronize()
        assert got_dt.dtype == torch.float32 and got_da.dtype == torch.float32
        _check(f"cumsum.dt[{softplus},{use_bias},{limit}]", got_dt, want_dt, 2e-6, 1e-9)
        _check(f"cumsum.dA_cumsum[{softplus},{use_bias},{limit}]", got_da, want_da, 1e-5, 1e-6)


def test_chunk_cumsum_strided_dt_and_pipeline(ops, oracle):
    # dt as a strided slice of a packed projection, then the whole pipeline cumsum -> fused against the oracle
    d = oracle.make_inputs(1, b=2, L=1024, H=6, init=True)
    Q = d["cfg"]["Q"]
    raw = d["dt_raw"]
    packed = torch.zeros(raw.shape[0], raw.shape[1], raw.shape[2] + 10, dtype=raw.dtype)
    packed[..., 7:7 + raw.shape[2]] = raw
    view = _dev(packed)[..., 7:7 + raw.shape[2]]
    assert not view.is_contiguous()
    dA, dt = ops._chunk_cumsum_fwd(view, _dev(d["A"]), Q, dt_bias=_dev(d["dt_bias"]), dt_softplus=True)
    _check("cumsum.strided.dt", dt, d["dt"], 2e-6, 1e-9)
    _check("cumsum.strided.dA", dA, d["dA_cumsum"], 1e-5, 1e-6)
    out, fin = ops._fused_chunk_state_state_passing_fwd(_dev(d["B"]), _dev(d["x"]), dt, dA, torch.float32,
                                                        initial_states=_dev(d["initial_states"]))
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
    _check("pipeline.out", out, want_out)
    _check("pipeline.final", fin, want_fin)


# ------------------------------------------------------------------ dt preparation + fused path in one call
@pytest.mark.parametrize("kw", [
    dict(),                                              # chunk 256, dstate 128
    dict(L=1000, nseq=5),                                # ragged last chunk + packed sequences
    dict(Q=128, L=1024, N=64, H=8, G=2),                 # chunk 128, dstate 64, grouped B
    dict(dtype="fp32", L=512),                           # fp32 inputs
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()) or "base")
def test_fused_with_dt_preparation(ops, oracle, kw):
    # one call for cumsum -> fused: against the same composition of the oracle, and the dt / dA_cumsum it returns
    # against the library's stand-alone producer bit for bit
    base = dict(b=2, L=1024, H=6, G=1, init=True)
    base.update(kw)
    d = oracle.make_inputs(1, **base)
    Q = d["cfg"]["Q"]
    raw, A, bias, seq, init = d["dt_raw"], d["A"], d["dt_bias"], d["seq_idx"], d["initial_states"]
    for softplus, use_bias, limit in ((True, True, (0.0, float("inf"))), (False, False, (1e-3, 0.1))):
        b_ = bias if use_bias else None
        want_da, want_dt = oracle.chunk_cumsum_ref(raw, A, Q, dt_bias=b_, dt_softplus=softplus, dt_limit=limit)
        want_out, want_fin = oracle.fused_ref(d["B"], d["x"], want_dt, want_da, initial_states=init, seq_idx=seq)
        out, fin, dA, dt = ops._fused_cumsum_chunk_state_state_passing_fwd(
            _dev(d["B"]), _dev(d["x"]), _dev(raw), _dev(A), Q, torch.float32, dt_bias=_dev(b_), dt_softplus=softplus,
            dt_limit=limit, initial_states=_dev(init), seq_idx=_dev(seq))
        torch.cuda.synchronize()
        tag = f"prep+fused[{softplus}]"
        _check(tag + ".dt", dt, want_dt, 2e-6, 1e-9)
        _check(tag + ".dA_cumsum", dA, want_da, 1e-5, 1e-6)
        _check(tag + ".out", out, want_out)
        _check(tag + ".final", fin, want_fin)
        dA2, dt2 = ops._chunk_cumsum_fwd(_dev(raw), _dev(A), Q, dt_bias=_dev(b_), dt_softplus=softplus, dt_limit=limit)
        out2, fin2 = ops._fused_chunk_state_state_passing_fwd(_dev(d["B"]), _dev(d["x"]), dt2, dA2, torch.float32,
                                                              initial_states=_dev(init), seq_idx=_dev(seq))
        torch.cuda.synchronize()
        assert torch.equal(dt2, dt) and torch.equal(dA2, dA), tag
        assert torch.equal(out2, out) and torch.equal(fin2, fin), tag


# ------------------------------------------------------------------ the consumer of the passed states
@pytest.mark.parametrize("kw", [
    dict(),                                              # chunk 256, dstate 128, headdim 64: matrix-core kernel
    dict(L=1000, nseq=5),                                # ragged last chunk + packed sequences
    dict(Q=128, L=1024, H=8, G=4),                       # chunk 128, grouped C
    dict(Q=64, L=512, N=64),                             # chunk 64, dstate 64
    dict(P=32, H=4),                                     # headdim 32: two row blocks per item
    dict(P=128, H=4),                                    # headdim 128: two items per head
    dict(L=300, H=3, P=40, N=24, G=1, Q=64),             # nothing aligned: plain FMA kernel
    dict(dtype="fp16"),                                  # fp16 C: plain FMA kernel
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()) or "base")
@pytest.mark.parametrize("kernel", [1, 2])
def test_chunk_scan_states(ops, oracle, kw, kernel):
    # kernel: both matrix-core decompositions in turn (the library picks by problem size; shapes that the forced
    # one does not take fall through to the other or to the plain kernel)
    base = dict(b=2, L=1024, H=6, G=1, init=True)
    base.update(kw)
    old = ops.set_scan_kernel(kernel)
    try:
        _scan_states_case(ops, oracle, base)
    finally:
        ops.set_scan_kernel(old)


def _scan_states_case(ops, oracle, base):
    d = oracle.make_inputs(1, **base)
    C, seq, dA = d["C"], d["seq_idx"], d["dA_cumsum"]
    prev, _ = oracle.fused_ref(d["B"], d["x"], d["dt"], dA, initial_states=d["initial_states"], seq_idx=seq)
    want = oracle.chunk_scan_states_ref(C, prev, dA, seq_idx=seq)
    Cd, pd, dAd, sd = _dev(C), _dev(prev), _dev(dA), _dev(seq)
    print(f"[scan_states] C{tuple(C.shape)} {C.dtype} states{tuple(prev.shape)}", flush=True)
    y = ops._chunk_scan_states_fwd(Cd, pd, dAd, seq_idx=sd, out_dtype=torch.float32)
    torch.cuda.synchronize()
    assert y.dtype == torch.float32 and y.shape == want.shape
    _check("scan_states.f32", y, want)
    # default output type follows C (the reference's out follows x); judged at the reference's own tolerance
    yb = ops._chunk_scan_states_fwd(Cd, pd, dAd, seq_idx=sd)
    assert yb.dtype == C.dtype
    _check("scan_states.lowp", yb.float(), want, 1e-2, 1e-2)
    # accumulate: added to what the output holds, on a strided view of a wider buffer
    wide = torch.randn(want.shape[0], want.shape[1], want.shape[2], want.shape[3] + 8, generator=torch.Generator().manual_seed(1))
    view = _dev(wide)[..., 8:]
    got = ops._chunk_scan_states_fwd(Cd, pd, dAd, seq_idx=sd, out=view, accumulate=True)
    torch.cuda.synchronize()
    assert got.data_ptr() == view.data_ptr()
    _check("scan_states.accumulate", view, want + wide[..., 8:])
    # bf16 passed states (what the reference's scan is handed, main.py:85-100): judged against the oracle on the same
    # rounded states -- the kernel then does what the fp32 one does, minus the rounding of its own hi + lo split
    prev16 = prev.to(torch.bfloat16)
    want16 = oracle.chunk_scan_states_ref(C, prev16.float(), dA, seq_idx=seq)
    y16 = ops._chunk_scan_states_fwd(Cd, _dev(prev16), dAd, seq_idx=sd, out_dtype=torch.float32)
    torch.cuda.synchronize()
    _check("scan_states.bf16states", y16, want16)
    got = ops._chunk_scan_states_fwd(Cd, _dev(prev16), dAd, seq_idx=sd, out=view, accumulate=True)
    torch.cuda.synchronize()
    _check("scan_states.bf16states.accumulate", view, want + want16 + wide[..., 8:], 2e-3, 2e-3)


def test_chunk_scan_states_cfg2_row(ops, oracle):
    # one batch row of the Mamba2-2.7B layer shape at full sequence length, states produced by the fused kernel
    d = oracle.make_inputs(2, b=1)
    dA = d["dA_cumsum"]
    xd, Bd, dtd, dAd, Cd = map(_dev, (d["x"], d["B"], d["dt"], dA, d["C"]))
    prev, _ = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, torch.float32, initial_states=_dev(d["initial_states"]))
    y = ops._chunk_scan_states_fwd(Cd, prev, dAd, out_dtype=torch.float32)
    torch.cuda.synchronize()
    want = oracle.chunk_scan_states_ref(d["C"], prev.cpu(), dA)
    _check("scan_states.cfg2row", y, want)
    # size-independent property: linear in C -- exact for a power of two, up to terms at the denormal threshold
    # (states of fast-decaying heads are that small, and the matrix cores flush what falls below it)
    y2 = ops._chunk_scan_states_fwd(Cd * 2.0, prev, dAd, out_dtype=torch.float32)
    torch.cuda.synchronize()
    err = float((y2 - y * 2.0).abs().max())
    print(f"[scan_states.linearity] max_abs={err:.3e}", flush=True)
    assert err <= 1e-30


@pytest.mark.timeout(900)
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_chunk_scan_states_long_grouped(ops, oracle, out_dtype):
    # The long grouped configuration at full size: seqlen * row pitch of y is 4.3 GB in fp32, past what one 32-bit
    # buffer descriptor reaches, so C and y are addressed chunk by chunk.  The states come from the fused call; two
    # heads of different groups are compared with the oracle, and the call must have run on the matrix-core kernels
    # (the element-per-thread fallback would take seconds).
    d = oracle.make_inputs(4)
    dA = d["dA_cumsum"]
    xd, Bd, dtd, dAd, Cd = map(_dev, (d["x"], d["B"], d["dt"], dA, d["C"]))
    prev, _ = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, torch.float32)
    del xd, Bd, dtd
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    y = ops._chunk_scan_states_fwd(Cd, prev, dAd, out_dtype=out_dtype)       # warm-up
    ev[0].record()
    y = ops._chunk_scan_states_fwd(Cd, prev, dAd, out_dtype=out_dtype)
    ev[1].record()
    torch.cuda.synchronize()
    ms = ev[0].elapsed_time(ev[1])
    print(f"[scan_states.cfg4.{out_dtype}] {ms * 1e3:.0f} us", flush=True)
    assert ms < 20.0, "the matrix-core kernels take a few milliseconds at this size"
    ratio = d["x"].shape[2] // d["B"].shape[2]
    lowp = out_dtype != torch.float32
    for h in (5, 127):
        g = h // ratio
        want = oracle.chunk_scan_states_ref(d["C"][:, :, g:g + 1], prev[:, :, h:h + 1].cpu(), dA[:, h:h + 1])
        _check(f"scan_states.cfg4.h{h}", y[:, :, h:h + 1], want, *((1e-2, 1e-2) if lowp else (RTOL, ATOL)))


# ------------------------------------------------------------------ the path inside a whole SSD forward
@pytest.mark.parametrize("kw", [dict(), dict(nseq=4, L=900, init=True)], ids=["plain", "varlen-ragged-init"])
def test_whole_ssd_forward_with_library_kernels(ops, oracle, kw):
    # main.py:78-103: cumsum -> fused chunk state + state passing run on the GPU through the library, the two
    # stages after them (bmm, chunk scan) are the oracle's restatements; the result is compared with the
    # token-serial selective scan, which knows nothing about chunks.
    base = dict(b=1, L=1024, H=4, G=2)
    base.update(kw)
    d = oracle.make_inputs(1, **base)
    Q = d["cfg"]["Q"]
    g = torch.Generator().manual_seed(11)
    D = torch.randn(d["x"].shape[2], generator=g)
    seq, init = d["seq_idx"], d["initial_states"]
    dA, dt = ops._chunk_cumsum_fwd(_dev(d["dt_raw"]), _dev(d["A"]), Q, dt_bias=_dev(d["dt_bias"]), dt_softplus=True)
    states, final = ops._fused_chunk_state_state_passing_fwd_globalbar(_dev(d["B"]), _dev(d["x"]), dt, dA, torch.float32,
                                                                       initial_states=_dev(init), seq_idx=_dev(seq))
    torch.cuda.synchronize()
    cb = oracle.bmm_chunk_ref(d["C"], d["B"], Q, seq_idx=seq)
    y, _ = oracle.chunk_scan_ref(cb, d["x"], dt.cpu(), dA.cpu(), d["C"], states.cpu(), D=D, seq_idx=seq)
    y64, h64 = oracle.token_scan_ref(d["x"], d["B"], d["C"], d["dt_tok"], d["A"], D=D, initial_states=init, seq_idx=seq)
    _check("forward.y", y, y64.float())
    _check("forward.final", final, h64.float())
