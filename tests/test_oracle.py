"""Pins the CPU oracle (oracle/ssd_oracle.py and the plain-C oracle/ssd_oracle.c) by mathematics.

The reference ships no stored answers and no CPU implementation, so the checks below are chosen so that a
plausible restatement mistake (dropped dt factor, wrong sign of the exponent, decay indexed at lim-1 instead
of Q-1, transposed p/n, group mapping off, exclusive vs inclusive scan, seq reset applied to the wrong chunk)
fails at least one of them."""
import math

import pytest
import torch

torch.manual_seed(0)


def _rand_case(b=2, L=48, H=4, P=4, N=6, G=2, Q=16, seed=1, ragged=False, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    if ragged:
        L = L - 5
    x = torch.randn(b, L, H, P, generator=g).to(dtype)
    B = torch.randn(b, L, G, N, generator=g).to(dtype)
    A = -torch.exp(torch.empty(H).uniform_(0.0, math.log(16.0), generator=g))
    dt_raw = torch.empty(b, L, H).uniform_(0.001, 0.1, generator=g)
    return x, B, A, dt_raw, Q


# ----------------------------------------------------------------------------- chunk cumsum
def test_chunk_cumsum_layout_and_padding(oracle):
    x, B, A, dt_raw, Q = _rand_case(ragged=True)
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    b, L, H = dt_raw.shape
    C = math.ceil(L / Q)
    assert dt.shape == dAcs.shape == (b, H, C, Q)
    for c in range(C):
        lim = min(Q, L - c * Q)
        torch.testing.assert_close(dt[:, :, c, :lim], dt_raw[:, c * Q:c * Q + lim].permute(0, 2, 1))
        assert (dt[:, :, c, lim:] == 0).all()
    # brute-force running sum
    run = torch.zeros(b, H)
    for k in range(Q):
        run = run + dt[:, :, 1, k] * A
        torch.testing.assert_close(dAcs[:, :, 1, k], run)


def test_chunk_cumsum_activation(oracle):
    dt_raw = torch.tensor([[[-3.0, 0.5, 19.0, 25.0]]])
    A = -torch.ones(4)
    bias = torch.tensor([0.1, 0.2, 0.3, 0.4])
    _, dt = oracle.chunk_cumsum_ref(dt_raw, A, 1, dt_bias=bias, dt_softplus=True, dt_limit=(0.05, 22.0))
    v = dt_raw[0, 0] + bias
    exp = torch.where(v <= 20, torch.log1p(torch.exp(v)), v).clamp(0.05, 22.0)
    torch.testing.assert_close(dt[0, :, 0, 0], exp)
    assert dt[0, 3, 0, 0] == 22.0 and dt[0, 0, 0, 0] == pytest.approx(max(math.log1p(math.exp(-2.9)), 0.05))


# ----------------------------------------------------------------------------- chunk state
def test_chunk_state_closed_form_geometric(oracle, oracle_c):
    # x = 1, B = 1, dt = d, A = a  =>  every entry = d * sum_{j<Q} exp(a d j)
    b, L, H, P, N, Q = 1, 64, 2, 3, 5, 32
    d, a = 0.05, -2.0
    x, B = torch.ones(b, L, H, P), torch.ones(b, L, 1, N)
    dAcs, dt = oracle.chunk_cumsum_ref(torch.full((b, L, H), d), torch.full((H,), a), Q)
    want = d * (1 - math.exp(a * d * Q)) / (1 - math.exp(a * d))
    for st in (oracle.chunk_state_ref(B, x, dt, dAcs), oracle_c.chunk_state(B, x, dt, dAcs)):
        torch.testing.assert_close(st, torch.full_like(st, want), rtol=1e-5, atol=1e-6)


def test_chunk_state_A_zero_is_plain_weighted_gram(oracle, oracle_c):
    x, B, A, dt_raw, Q = _rand_case(G=1)
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, torch.zeros_like(A), Q)
    b, L, H, P = x.shape
    C = L // Q
    xs = (x * dt_raw[..., None]).reshape(b, C, Q, H, P)
    want = torch.einsum("bcqhp,bcqn->bchpn", xs, B[:, :, 0].reshape(b, C, Q, -1))
    for st in (oracle.chunk_state_ref(B, x, dt, dAcs), oracle_c.chunk_state(B, x, dt, dAcs)):
        torch.testing.assert_close(st, want, rtol=1e-5, atol=1e-6)


def test_chunk_state_one_hot_picks_single_weight(oracle, oracle_c):
    # x and B one-hot in (token k0, p0) / (token k0, n0): the only non-zero entry is w[k0] at (p0, n0),
    # and it sits at [p0, n0] (not transposed).
    b, L, H, P, N, Q = 1, 32, 1, 3, 4, 16
    g = torch.Generator().manual_seed(3)
    dt_raw = torch.empty(b, L, H).uniform_(0.01, 0.1, generator=g)
    A = torch.tensor([-3.0])
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    k0, p0, n0, c0 = 5, 2, 1, 1
    x, B = torch.zeros(b, L, H, P), torch.zeros(b, L, 1, N)
    x[0, c0 * Q + k0, 0, p0] = 2.0
    B[0, c0 * Q + k0, 0, n0] = 3.0
    # decay from token k0 to the END of the chunk, times dt at k0
    w = math.exp(float((dt_raw[0, c0 * Q + k0 + 1:(c0 + 1) * Q, 0] * A[0]).sum())) * float(dt_raw[0, c0 * Q + k0, 0])
    for st in (oracle.chunk_state_ref(B, x, dt, dAcs), oracle_c.chunk_state(B, x, dt, dAcs)):
        want = torch.zeros_like(st)
        want[0, c0, 0, p0, n0] = 6.0 * w
        torch.testing.assert_close(st, want, rtol=1e-5, atol=1e-7)


def test_chunk_state_brute_force_groups_and_ragged(oracle, oracle_c):
    x, B, A, dt_raw, Q = _rand_case(ragged=True)
    b, L, H, P = x.shape
    G, N = B.shape[2:]
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    C = dt.shape[2]
    want = torch.zeros(b, C, H, P, N, dtype=torch.float64)
    for bi in range(b):
        for c in range(C):
            for h in range(H):
                for k in range(min(Q, L - c * Q)):
                    t = c * Q + k
                    dec = math.exp(sum(float(dt_raw[bi, u, h]) * float(A[h]) for u in range(t + 1, min((c + 1) * Q, L))))
                    want[bi, c, h] += dec * float(dt_raw[bi, t, h]) * torch.outer(x[bi, t, h].double(), B[bi, t, h // (H // G)].double())
    for st in (oracle.chunk_state_ref(B, x, dt, dAcs), oracle_c.chunk_state(B, x, dt, dAcs)):
        torch.testing.assert_close(st.double(), want, rtol=2e-5, atol=2e-6)
    st64 = oracle.chunk_state_ref(B, x, dt, dAcs, compute_dtype=torch.float64)
    torch.testing.assert_close(st64, want, rtol=1e-6, atol=1e-7)


def test_chunk_state_group_sharing(oracle):
    # heads of one group with identical x / dt / A give identical states
    x, B, A, dt_raw, Q = _rand_case(H=4, G=2)
    x[:, :, 1] = x[:, :, 0]
    dt_raw[:, :, 1] = dt_raw[:, :, 0]
    A[1] = A[0]
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    st = oracle.chunk_state_ref(B, x, dt, dAcs)
    assert torch.equal(st[:, :, 0], st[:, :, 1])
    assert not torch.allclose(st[:, :, 0], st[:, :, 2])


def test_chunk_state_seq_idx_masks_other_sequences(oracle, oracle_c):
    x, B, A, dt_raw, Q = _rand_case(b=1, L=32, Q=16, G=1)
    seq = torch.zeros(1, 32, dtype=torch.int32)
    seq[0, 10:] = 1          # boundary inside chunk 0; chunk 1 is entirely sequence 1
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    x0 = x.clone()
    x0[0, :10] = 0           # dropping the earlier sequence's tokens by hand must be equivalent
    want = oracle.chunk_state_ref(B, x0, dt, dAcs)
    for st in (oracle.chunk_state_ref(B, x, dt, dAcs, seq_idx=seq), oracle_c.chunk_state(B, x, dt, dAcs, seq_idx=seq)):
        torch.testing.assert_close(st, want, rtol=1e-5, atol=1e-6)
    assert not torch.allclose(want[0, 0], oracle.chunk_state_ref(B, x, dt, dAcs)[0, 0])


def test_chunk_state_clamp_only_matters_for_increasing_cumsum(oracle, oracle_c):
    x, B, A, dt_raw, Q = _rand_case(G=1)
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    a = oracle.chunk_state_ref(B, x, dt, dAcs, clamp=True)
    torch.testing.assert_close(a, oracle.chunk_state_ref(B, x, dt, dAcs, clamp=False))
    dAcs_pos, _ = oracle.chunk_cumsum_ref(dt_raw, -A, Q)       # increasing cumsum: exponent positive -> clamped to 0
    c1 = oracle.chunk_state_ref(B, x, dt, dAcs_pos, clamp=True)
    c0 = oracle.chunk_state_ref(B, x, dt, dAcs_pos, clamp=False)
    plain = oracle.chunk_state_ref(B, x, dt, torch.zeros_like(dAcs))
    torch.testing.assert_close(c1, plain)
    assert not torch.allclose(c0, c1)
    torch.testing.assert_close(oracle_c.chunk_state(B, x, dt, dAcs_pos, clamp=False), c0, rtol=1e-5, atol=1e-5)


# ----------------------------------------------------------------------------- state passing
def test_state_passing_closed_form(oracle, oracle_c):
    # constant new state T, constant decay r:  s_c = T (1 - r^{c+1})/(1-r) + r^{c+1} s_init
    b, C, H, dim = 2, 7, 3, 5
    T = torch.randn(1, 1, H, dim).expand(b, C, H, dim).contiguous()
    dA = torch.full((b, H, C), -0.3)
    init = torch.randn(b, H, dim)
    r = math.exp(-0.3)
    for out, fin in (oracle.state_passing_ref(T, dA, init), oracle_c.state_passing(T, dA, init)):
        assert torch.equal(out[:, 0], init)
        for c in range(C):
            want = T[:, 0] * (1 - r ** (c + 1)) / (1 - r) + r ** (c + 1) * init
            got = out[:, c + 1] if c < C - 1 else fin
            torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_state_passing_zero_decay_is_exclusive_cumsum(oracle, oracle_c):
    st = torch.randn(2, 6, 3, 4)
    dA = torch.zeros(2, 3, 6)
    cs = torch.cumsum(st, dim=1)
    for out, fin in (oracle.state_passing_ref(st, dA), oracle_c.state_passing(st, dA)):
        assert (out[:, 0] == 0).all()
        torch.testing.assert_close(out[:, 1:], cs[:, :-1])
        torch.testing.assert_close(fin, cs[:, -1])


def test_state_passing_strong_decay_forgets(oracle):
    st = torch.randn(1, 4, 2, 3)
    out, fin = oracle.state_passing_ref(st, torch.full((1, 2, 4), -200.0), torch.randn(1, 2, 3))
    torch.testing.assert_close(out[:, 1:], st[:, :-1])
    torch.testing.assert_close(fin, st[:, -1])


def test_state_passing_seq_idx_reset_and_prev_starts_at_zero(oracle, oracle_c):
    b, C, H, dim, Q = 1, 4, 2, 3, 8
    st = torch.randn(b, C, H, dim)
    dA = -torch.rand(b, H, C)
    init = torch.randn(b, H, dim)
    seq = torch.zeros(1, C * Q, dtype=torch.int32)
    seq[0, 2 * Q - 3:] = 1            # chunk 1 ends in sequence 1 -> carried state dropped at c = 1
    for out, fin in (oracle.state_passing_ref(st, dA, init, seq, Q), oracle_c.state_passing(st, dA, init, seq, Q)):
        torch.testing.assert_close(out[:, 1], torch.exp(dA[:, :, 0])[..., None] * init + st[:, 0])
        torch.testing.assert_close(out[:, 2], st[:, 1])
        torch.testing.assert_close(out[:, 3], torch.exp(dA[:, :, 2])[..., None] * st[:, 1] + st[:, 2])
    seq1 = torch.ones(1, C * Q, dtype=torch.int32)     # ids start at 1: the initial state is dropped (prev = 0)
    out, _ = oracle.state_passing_ref(st, dA, init, seq1, Q)
    torch.testing.assert_close(out[:, 1], st[:, 0])


def test_state_passing_out_dtype_and_final_fp32(oracle):
    st = torch.randn(1, 3, 2, 4)
    out, fin = oracle.state_passing_ref(st, -torch.rand(1, 2, 3), out_dtype=torch.bfloat16)
    assert out.dtype == torch.bfloat16 and fin.dtype == torch.float32


# ----------------------------------------------------------------------------- composed path
@pytest.mark.parametrize("ragged", [False, True])
@pytest.mark.parametrize("with_init", [False, True])
def test_fused_equals_token_recurrence(oracle, oracle_c, ragged, with_init):
    x, B, A, dt_raw, Q = _rand_case(ragged=ragged)
    b, L, H, P = x.shape
    N = B.shape[-1]
    init = torch.randn(b, H, P, N) if with_init else None
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    out, fin = oracle.fused_ref(B, x, dt, dAcs, initial_states=init)
    out64, fin64 = oracle.token_recurrence_ref(x, B, dt_raw, A, Q, init)
    torch.testing.assert_close(out.double(), out64, rtol=2e-5, atol=2e-6)
    torch.testing.assert_close(fin.double(), fin64, rtol=2e-5, atol=2e-6)
    outc, finc = oracle_c.token_recurrence(x, B, dt_raw, A, Q, init)
    torch.testing.assert_close(outc, out64, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(finc, fin64, rtol=1e-10, atol=1e-12)
    # fp64 chunked evaluation agrees much more tightly: the difference above is fp32 roundoff only
    o64, f64 = oracle.fused_ref(B, x, dt.double(), dAcs.double(), initial_states=init, compute_dtype=torch.float64)
    torch.testing.assert_close(o64, out64, rtol=1e-5, atol=1e-7)   # dt/dAcs were rounded to fp32 by the producer


def test_chunk_size_invariance(oracle):
    x, B, A, dt_raw, _ = _rand_case(L=64)
    finals, outs = [], {}
    for Q in (8, 16, 32):
        dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
        out, fin = oracle.fused_ref(B, x, dt, dAcs)
        finals.append(fin)
        outs[Q] = out
    torch.testing.assert_close(finals[0], finals[1], rtol=2e-5, atol=2e-6)
    torch.testing.assert_close(finals[0], finals[2], rtol=2e-5, atol=2e-6)
    torch.testing.assert_close(outs[8][:, ::4], outs[32], rtol=2e-5, atol=2e-6)
    torch.testing.assert_close(outs[16][:, ::2], outs[32], rtol=2e-5, atol=2e-6)


def test_varlen_equals_concatenation_of_solo_runs(oracle, oracle_c):
    b, H, P, N, G, Q = 1, 4, 4, 6, 2, 16
    lens = [23, 9, 40, 24]      # boundaries inside chunks, a sequence shorter than a chunk, total 96 = 6 chunks
    L = sum(lens)
    x, B, A, dt_raw, _ = _rand_case(b=b, L=L, H=H, P=P, N=N, G=G, Q=Q, seed=7)
    seq = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens)).to(torch.int32)[None]
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    out, fin = oracle.fused_ref(B, x, dt, dAcs, seq_idx=seq)
    out_t, fin_t = oracle.token_recurrence_ref(x, B, dt_raw, A, Q, seq_idx=seq)
    torch.testing.assert_close(out.double(), out_t, rtol=2e-5, atol=2e-6)
    torch.testing.assert_close(fin.double(), fin_t, rtol=2e-5, atol=2e-6)
    out_c, fin_c = oracle_c.token_recurrence(x, B, dt_raw, A, Q, seq_idx=seq)
    torch.testing.assert_close(out_c, out_t, rtol=1e-10, atol=1e-12)
    # solo runs: state of the sequence that owns token cQ-1, evaluated alone from a zero state
    start = 0
    for i, n in enumerate(lens):
        sl = slice(start, start + n)
        _, h = oracle.token_recurrence_ref(x[:, sl], B[:, sl], dt_raw[:, sl], A, 10 ** 6)
        if i == len(lens) - 1:
            torch.testing.assert_close(fin.double(), h, rtol=2e-5, atol=2e-6)
        for c in range(1, L // Q):
            t = c * Q - 1
            if start <= t < start + n:
                _, hc = oracle.token_recurrence_ref(x[:, start:t + 1], B[:, start:t + 1], dt_raw[:, start:t + 1], A, 10 ** 6)
                torch.testing.assert_close(out[:, c].double(), hc, rtol=2e-5, atol=2e-6)
        start += n


def test_linearity_and_initial_state_decay(oracle):
    x, B, A, dt_raw, Q = _rand_case(G=1)
    b, L, H, P = x.shape
    N = B.shape[-1]
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    init = torch.randn(b, H, P, N)
    o0, f0 = oracle.fused_ref(B, x, dt, dAcs)
    o1, f1 = oracle.fused_ref(B, x, dt, dAcs, initial_states=init)
    total = torch.exp((dt_raw * A).sum(dim=1))                     # (b,H)
    torch.testing.assert_close(f1 - f0, total[..., None, None] * init, rtol=1e-4, atol=1e-6)
    o2, f2 = oracle.fused_ref(B, 2.0 * x, dt, dAcs)
    torch.testing.assert_close(f2, 2.0 * f0, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(o2, 2.0 * o0, rtol=1e-5, atol=1e-6)


def test_ragged_equals_zero_padded(oracle):
    x, B, A, dt_raw, Q = _rand_case(ragged=True)
    b, L, H, P = x.shape
    pad = (-L) % Q
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    o, f = oracle.fused_ref(B, x, dt, dAcs)
    xp = torch.nn.functional.pad(x, (0, 0, 0, 0, 0, pad), value=7.0)      # garbage x in the padding...
    Bp = torch.nn.functional.pad(B, (0, 0, 0, 0, 0, pad), value=-3.0)
    dtp = torch.nn.functional.pad(dt_raw, (0, 0, 0, pad), value=0.0)      # ...but dt = 0 there
    dAcs2, dt2 = oracle.chunk_cumsum_ref(dtp, A, Q)
    o2, f2 = oracle.fused_ref(Bp, xp, dt2, dAcs2)
    torch.testing.assert_close(o, o2)
    torch.testing.assert_close(f, f2)


def test_fused_states_side_effect_and_unfused_composition(oracle, oracle_c):
    x, B, A, dt_raw, Q = _rand_case()
    b, L, H, P = x.shape
    N = B.shape[-1]
    dAcs, dt = oracle.chunk_cumsum_ref(dt_raw, A, Q)
    buf = torch.empty(b, L // Q, H, P, N)
    out, fin = oracle.fused_ref(B, x, dt, dAcs, states=buf)
    st = oracle.chunk_state_ref(B, x, dt, dAcs)
    assert torch.equal(buf, st)
    o2, f2 = oracle.state_passing_ref(st.flatten(-2), dAcs[..., -1])
    assert torch.equal(out, o2.reshape(out.shape)) and torch.equal(fin, f2.reshape(fin.shape))
    o3, f3 = oracle_c.state_passing(oracle_c.chunk_state(B, x, dt, dAcs).flatten(-2), dAcs[..., -1])
    torch.testing.assert_close(o3.reshape(out.shape), out, rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------------------- input recipe
def test_make_inputs_shapes_and_distributions(oracle):
    d = oracle.make_inputs(3, L=4096, H=4, nseq=5)
    assert d["x"].dtype == torch.bfloat16 and d["x"].shape == (1, 4096, 4, 64)
    assert d["dt"].shape == d["dA_cumsum"].shape == (1, 4, 16, 256)
    assert d["seq_idx"].dtype == torch.int32 and int(d["seq_idx"].max()) == 4 and int(d["seq_lens"].sum()) == 4096
    assert (d["seq_idx"][0, 1:] >= d["seq_idx"][0, :-1]).all()
    assert 0.9e-3 < float(d["dt"].min()) and float(d["dt"].max()) < 1.1e-1
    assert (d["A"] <= -1).all() and (d["A"] >= -16).all()
    assert (d["dA_cumsum"][..., 1:] <= d["dA_cumsum"][..., :-1]).all()
    d2 = oracle.make_inputs(3, L=4096, H=4, nseq=5)
    assert torch.equal(d["x"], d2["x"]) and torch.equal(d["dt"], d2["dt"])
    c2 = oracle.CONFIGS[2]
    assert oracle.algorithmic_bytes(c2) == 721_420_288 and oracle.algorithmic_flops(c2) == 43_117_445_120


# ---------------------------------------------------------------- the callers either side of the path
def _ssd_forward_chunked(o, d, Cm, D, z, Q):
    """main.py:78-103 with the oracle's restatements: cumsum -> fused -> bmm -> chunk scan."""
    dA, dt = o.chunk_cumsum_ref(d["dt_raw"], d["A"], Q, dt_bias=d["dt_bias"], dt_softplus=True)
    states, final = o.fused_ref(d["B"], d["x"], dt, dA, initial_states=d["initial_states"], seq_idx=d["seq_idx"])
    cb = o.bmm_chunk_ref(Cm, d["B"], Q, seq_idx=d["seq_idx"])
    out, out_x = o.chunk_scan_ref(cb, d["x"], dt, dA, Cm, states, D=D, z=z, seq_idx=d["seq_idx"])
    return out, out_x, final


@pytest.mark.parametrize("kw", [
    dict(),
    dict(nseq=3, L=200),                       # packed sequences + ragged last chunk
    dict(G=2, init=True),                      # grouped B / C, initial states
], ids=["base", "varlen-ragged", "groups-init"])
def test_whole_forward_equals_token_serial_scan(oracle, kw):
    o = oracle
    base = dict(b=2, L=192, H=4, P=8, N=16, G=1, Q=64, dtype="fp32")
    base.update(kw)
    d = o.make_inputs(1, **base)
    g = torch.Generator().manual_seed(7)
    D = torch.randn(4, generator=g)
    z = torch.randn(d["x"].shape, generator=g)
    out, out_x, final = _ssd_forward_chunked(o, d, d["C"], D, z, 64)
    y64, h64 = o.token_scan_ref(d["x"], d["B"], d["C"], d["dt_tok"], d["A"], D=D, initial_states=d["initial_states"],
                                seq_idx=d["seq_idx"])
    assert torch.allclose(out_x.double(), y64, rtol=1e-4, atol=1e-5)
    assert torch.allclose(out.double(), y64 * z.double() * torch.sigmoid(z.double()), rtol=1e-4, atol=1e-5)
    assert torch.allclose(final.double(), h64, rtol=1e-4, atol=1e-5)
    # chunk-size invariance of the whole forward
    out2, _, final2 = _ssd_forward_chunked(o, d, d["C"], D, z, 32)
    assert torch.allclose(out2, out, rtol=1e-4, atol=1e-5) and torch.allclose(final2, final, rtol=1e-4, atol=1e-5)


def test_bmm_chunk_brute_force_and_masks(oracle):
    o = oracle
    g = torch.Generator().manual_seed(3)
    a = torch.randn(1, 10, 2, 3, generator=g)
    b = torch.randn(1, 10, 2, 3, generator=g)
    seq = torch.tensor([[0, 0, 0, 1, 1, 1, 1, 2, 2, 2]], dtype=torch.int32)
    out = o.bmm_chunk_ref(a, b, 4, seq_idx=seq)          # 3 chunks, the last one ragged (2 tokens)
    assert out.shape == (1, 3, 2, 4, 4)
    for c in range(3):
        for gi in range(2):
            for m in range(4):
                for n in range(4):
                    tm, tn = 4 * c + m, 4 * c + n
                    want = 0.0
                    if tm < 10 and tn < 10 and seq[0, tm] == seq[0, tn]:
                        want = float((a[0, tm, gi] * b[0, tn, gi]).sum())
                    assert abs(float(out[0, c, gi, m, n]) - want) < 1e-5, (c, gi, m, n)


def test_chunk_scan_special_cases(oracle):
    o = oracle
    b, L, H, P, N, Q = 1, 8, 2, 3, 4, 4
    g = torch.Generator().manual_seed(5)
    x = torch.randn(b, L, H, P, generator=g)
    C = torch.randn(b, L, 1, N, generator=g)
    states = torch.randn(b, 2, H, P, N, generator=g)
    zeros = torch.zeros(b, H, 2, Q)
    # dt = 0 and dA_cumsum = 0: no intra-chunk term, unit decay -> y[m] = C[m] . states[c]
    cb = torch.randn(b, 2, 1, Q, Q, generator=g)
    y, none = o.chunk_scan_ref(cb, x, zeros, zeros, C, states)
    assert none is None
    want = torch.einsum("bcmn,bchpn->bcmhp", C[:, :, 0].reshape(b, 2, Q, N), states).reshape(b, L, H, P)
    assert torch.allclose(y, want, atol=1e-6)
    # states = 0, dA_cumsum = 0, dt = 1: y[m] = sum_{k<=m} cb[m,k] x[k]  (causal), plus D x
    ones = torch.ones(b, H, 2, Q)
    D = torch.tensor([0.5, -2.0])
    y, _ = o.chunk_scan_ref(cb, x, ones, zeros, C, torch.zeros_like(states), D=D)
    for c in range(2):
        for m in range(Q):
            want = sum(cb[0, c, 0, m, k] * x[0, c * Q + k] for k in range(m + 1)) + x[0, c * Q + m] * D[:, None]
            assert torch.allclose(y[0, c * Q + m], want, atol=1e-5)


def test_chunk_scan_states_is_the_state_half_of_the_chunk_scan(oracle):
    o = oracle
    # (1) with cb = 0 (no intra-chunk term, no D) the pinned chunk scan reduces to its state half: ragged last chunk,
    #     grouped C, packed sequences
    d = o.make_inputs(0, b=2, L=200, H=4, G=2, P=8, N=16, Q=64, nseq=3)
    g = torch.Generator().manual_seed(3)
    states = torch.randn(2, 4, 4, 8, 16, generator=g)
    cb0 = torch.zeros(2, 4, 2, 64, 64)
    for seq in (None, d["seq_idx"]):
        want, _ = o.chunk_scan_ref(cb0, d["x"], d["dt"], d["dA_cumsum"], d["C"], states, seq_idx=seq)
        got = o.chunk_scan_states_ref(d["C"], states, d["dA_cumsum"], seq_idx=seq)
        assert got.shape == want.shape and torch.allclose(got, want, rtol=1e-6, atol=1e-6)
    # (2) brute force on a tiny case, element by element, with the first chunk's sequence ids != 0 (scale 0 there:
    #     the previous id of chunk 0 is taken as 0) and a change of sequence inside chunk 1
    b, L, H, P, N, Q = 1, 6, 2, 2, 3, 4
    C = torch.randn(b, L, 1, N, generator=g)
    st = torch.randn(b, 2, H, P, N, generator=g)
    dA = -torch.rand(b, H, 2, Q, generator=g)
    seq = torch.tensor([[1, 1, 1, 1, 1, 2]], dtype=torch.int32)
    got = o.chunk_scan_states_ref(C, st, dA, seq_idx=seq)
    for l in range(L):
        c, m = divmod(l, Q)
        prev = int(seq[0, c * Q - 1]) if c else 0
        for h in range(H):
            for p in range(P):
                dot = sum(float(C[0, l, 0, n]) * float(st[0, c, h, p, n]) for n in range(N))
                want = dot * math.exp(float(dA[0, h, c, m])) if int(seq[0, l]) == prev else 0.0
                assert abs(float(got[0, l, h, p]) - want) < 1e-5, (l, h, p)
    assert float(got[0, :4].abs().max()) == 0.0 and float(got[0, 4].abs().max()) > 0 and float(got[0, 5].abs().max()) == 0.0
    # (3) linear in the states and in C
    got2 = o.chunk_scan_states_ref(2 * C, st * -0.5, dA, seq_idx=seq)
    assert torch.allclose(got2, -got, atol=1e-6)
