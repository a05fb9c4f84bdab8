"""CPU oracle for the Mamba2 SSD chunk-state + state-passing path.

TEST INFRASTRUCTURE ONLY.  Nothing that ships (the wrappers, the C-ABI library,
the HIP kernels) imports this file.  It is used by the tests, by the smoke check
and by the benchmark's ``cpu_baseline`` leg, and only as the checker.

It restates, in plain fp32/fp64 PyTorch on the CPU, what the reference's Triton
kernels compute.  The reference ships no CPU implementation and no stored
answers, so every function below is pinned by mathematics instead (closed
forms, brute force on tiny shapes, the token-serial recurrence, chunk-size
invariance, packed-vs-solo equivalence); those checks live in
``tests/test_oracle.py``.

Functions and the reference lines they follow
---------------------------------------------
chunk_cumsum_ref       kernels/ssd_chunk_state.py:33-79, 176-199
chunk_state_ref        kernels/ssd_chunk_state.py:97-173, 202-232
state_passing_ref      kernels/ssd_state_passing.py:27-84, 87-115
fused_ref              kernels/fused_globalbar.py:201-266, kernels/fused_concurrent.py:255-331
                       (same contract: chunk state followed by state passing)
bmm_chunk_ref          kernels/ssd_bmm.py:31-134   (the step before the chunk scan; outside the path, used to
chunk_scan_ref         kernels/ssd_chunk_scan.py:38-215   run the path inside a whole SSD forward, main.py:60-104)
chunk_scan_states_ref  kernels/ssd_chunk_scan.py:94-117   (the state-consuming half of the chunk scan alone)
token_scan_ref         no counterpart in the reference: token-serial y_t = C_t . h_t + D x_t in fp64, which pins
                       the chunked composition cumsum -> chunk state -> state passing -> bmm -> chunk scan.
token_recurrence_ref   no counterpart in the reference: an independent, chunk-free
                       evaluation of the same linear recurrence used to pin the two
                       chunked functions.
make_inputs            the five benchmark configurations' own seeded recipe.
make_reference_inputs  kernels/rand_data.py:4-25, the reference's only input recipe (as main.py:166 draws it): the same
                       shapes, element types and distributions from a CPU generator (the reference draws on the GPU,
                       so the bits differ; the value ranges -- dt in [0.5, 1), A in (-1, 0], no softplus -- do not).

Pin status: all functions pinned (see tests/test_oracle.py); none is "parity unpinned".
"""
import math

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------
# Stage before the path: dt activation + per-chunk cumulative sum (input producer)
# --------------------------------------------------------------------------------------
def chunk_cumsum_ref(dt, A, chunk_size, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """Follows kernels/ssd_chunk_state.py:65-79.  dt (b, L, H) -> (dA_cumsum, dt_out), both (b, H, C, Q) fp32."""
    batch, seqlen, nheads = dt.shape
    assert A.shape == (nheads,)
    nchunks = math.ceil(seqlen / chunk_size)
    d = dt.float()
    if dt_bias is not None:
        assert dt_bias.shape == (nheads,)
        d = d + dt_bias.float()[None, None, :]
    if dt_softplus:
        # softplus only below the threshold 20, identity above (:70)
        d = torch.where(d <= 20.0, torch.log1p(torch.exp(torch.clamp(d, max=20.0))), d)
    d = torch.clamp(d, min=dt_limit[0], max=dt_limit[1])
    pad = nchunks * chunk_size - seqlen
    if pad:
        d = F.pad(d, (0, 0, 0, pad))  # tokens past the end contribute dt = 0 (:74)
    d = d.reshape(batch, nchunks, chunk_size, nheads).permute(0, 3, 1, 2).contiguous()
    dA = d * A.float()[None, :, None, None]
    return torch.cumsum(dA, dim=-1), d


# --------------------------------------------------------------------------------------
# a2: chunk state
# --------------------------------------------------------------------------------------
def _chunk_weights(dt, dA_cumsum, seqlen, seq_idx, clamp):
    """w[b,h,c,k] of kernels/ssd_chunk_state.py:134-156 (fp32 in, same dtype out)."""
    batch, nheads, nchunks, Q = dt.shape
    last = dA_cumsum[..., Q - 1:Q]                      # index Q-1, not lim-1 (:134)
    expo = last - dA_cumsum
    if clamp:
        expo = torch.clamp(expo, max=0.0)               # min(.,0) of the unfused kernel (:153)
    w = torch.exp(expo) * dt
    pos = torch.arange(nchunks * Q).reshape(nchunks, Q)
    valid = (pos < seqlen)                              # k < chunk_size_limit (:139, :145-150)
    w = w * valid[None, None].to(w.dtype)
    if seq_idx is not None:
        pad = nchunks * Q - seqlen
        s = seq_idx.long()
        if pad:
            s = F.pad(s, (0, pad), value=-1)
        s = s.reshape(batch, nchunks, Q)
        lim = torch.clamp(torch.tensor(seqlen) - torch.arange(nchunks) * Q, max=Q)  # (C,)
        s_last = torch.gather(s, 2, (lim - 1).reshape(1, nchunks, 1).expand(batch, nchunks, 1))  # (:141)
        same = (s == s_last)                            # (b, C, Q)  (:156)
        w = w * same[:, None].to(w.dtype)
    return w


def chunk_state_ref(B, x, dt, dA_cumsum, seq_idx=None, states=None, states_in_fp32=True,
                    compute_dtype=torch.float32, clamp=True):
    """states[b,c,h,p,n] = sum_k x[b,cQ+k,h,p] * B[b,cQ+k,g(h),n] * w[b,h,c,k]  (kernels/ssd_chunk_state.py:114-173).

    Evaluated in ``compute_dtype`` (fp32 by default, fp64 for pinning) on the exact input values, i.e.
    without the reference's rounding of B*w to the input dtype (:158)."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, Q = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, nheads, nchunks, Q)
    assert dA_cumsum.shape == dt.shape
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
    w = _chunk_weights(dt.to(compute_dtype), dA_cumsum.to(compute_dtype), seqlen, seq_idx, clamp)
    pad = nchunks * Q - seqlen
    ratio = nheads // ngroups
    out = torch.empty(batch, nchunks, nheads, headdim, dstate, dtype=compute_dtype)
    for b in range(batch):
        xb = x[b].to(compute_dtype)
        Bb = B[b].to(compute_dtype)
        if pad:
            xb = F.pad(xb, (0, 0, 0, 0, 0, pad))
            Bb = F.pad(Bb, (0, 0, 0, 0, 0, pad))
        xb = xb.reshape(nchunks, Q, nheads, headdim)
        Bb = Bb.reshape(nchunks, Q, ngroups, dstate)
        for g in range(ngroups):                        # g = h // (H/G)  (:121)
            hs = slice(g * ratio, (g + 1) * ratio)
            xw = xb[:, :, hs, :] * w[b, hs].permute(1, 2, 0)[..., None]      # (C,Q,r,P)
            # (C, r*P, Q) @ (C, Q, N)
            lhs = xw.permute(0, 2, 3, 1).reshape(nchunks, ratio * headdim, Q)
            res = torch.bmm(lhs, Bb[:, :, g, :])
            out[b, :, hs] = res.reshape(nchunks, ratio, headdim, dstate)
    res_dtype = torch.float32 if states_in_fp32 else B.dtype
    if compute_dtype == torch.float64 and states is None:
        return out
    if states is not None:
        assert states.shape == (batch, nchunks, nheads, headdim, dstate)
        states.copy_(out)
        return states
    return out.to(res_dtype)


# --------------------------------------------------------------------------------------
# a4: state passing
# --------------------------------------------------------------------------------------
def state_passing_ref(states, dA_chunk_cumsum, initial_states=None, seq_idx=None, chunk_size=None,
                      out_dtype=None, compute_dtype=torch.float32):
    """Follows kernels/ssd_state_passing.py:61-84; states (b,C,H,dim) -> out (b,C,H,dim), final (b,H,dim) fp32."""
    batch, nchunks, nheads, dim = states.shape
    assert dA_chunk_cumsum.shape == (batch, nheads, nchunks)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, dim)
    if seq_idx is not None:
        assert chunk_size is not None
        seqlen = seq_idx.shape[-1]
        assert seq_idx.shape == (batch, seqlen)
    out_dtype = states.dtype if out_dtype is None else out_dtype
    out = torch.empty(batch, nchunks, nheads, dim, dtype=compute_dtype)
    s = (torch.zeros(batch, nheads, dim, dtype=compute_dtype) if initial_states is None
         else initial_states.to(compute_dtype).clone())
    out[:, 0] = s                                       # (:66)
    prev = torch.zeros(batch, dtype=torch.long)         # integer 0, not seq_idx[:,0]  (:68)
    final = None
    for c in range(nchunks):
        scale = torch.exp(dA_chunk_cumsum[:, :, c].to(compute_dtype))        # (b,H)  (:72)
        if seq_idx is not None:
            cur = seq_idx[:, min((c + 1) * chunk_size, seqlen) - 1].long()   # (:74)
            scale = torch.where((cur == prev)[:, None], scale, torch.zeros_like(scale))
            prev = cur
        s = scale[..., None] * s + states[:, c].to(compute_dtype)            # (:77)
        if c < nchunks - 1:
            out[:, c + 1] = s
        else:
            final = s
    if compute_dtype == torch.float64:
        return out, final
    return out.to(out_dtype), final.to(torch.float32)   # final is always fp32 (:99)


# --------------------------------------------------------------------------------------
# a5/a7: the fused entry = chunk state, then state passing on the flattened (p n) axis
# --------------------------------------------------------------------------------------
def fused_ref(B, x, dt, dA_cumsum, out_dtype=None, initial_states=None, seq_idx=None, states=None,
              states_in_fp32=True, compute_dtype=torch.float32, clamp=True):
    """Contract of kernels/fused_globalbar.py:201-266 (and fused_concurrent.py:255-331).

    Returns (out (b,C,H,P,N), final_states (b,H,P,N) fp32).  ``initial_states`` is 4-D (b,H,P,N) here.
    If ``states`` is given it receives the per-chunk states as a side effect.  The fused reference kernels
    drop the min(.,0) clamp (fused_globalbar.py:106); with non-increasing dA_cumsum both forms agree, and
    ``clamp`` selects which one is evaluated."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, Q = dt.shape
    dstate = B.shape[-1]
    st = chunk_state_ref(B, x, dt, dA_cumsum, seq_idx=seq_idx, states_in_fp32=states_in_fp32,
                         compute_dtype=compute_dtype, clamp=clamp)
    if states is not None:
        assert states.shape == st.shape
        states.copy_(st)
    if initial_states is not None:
        assert initial_states.shape == (batch, nheads, headdim, dstate)
    init = None if initial_states is None else initial_states.reshape(batch, nheads, headdim * dstate)
    out_dtype = st.dtype if out_dtype is None else out_dtype
    out, final = state_passing_ref(st.reshape(batch, nchunks, nheads, headdim * dstate), dA_cumsum[..., -1],
                                   initial_states=init, seq_idx=seq_idx, chunk_size=Q, out_dtype=out_dtype,
                                   compute_dtype=compute_dtype)
    return (out.reshape(batch, nchunks, nheads, headdim, dstate),
            final.reshape(batch, nheads, headdim, dstate))


# --------------------------------------------------------------------------------------
# Independent pin: the chunk-free, token-serial recurrence (fp64)
# --------------------------------------------------------------------------------------
def token_recurrence_ref(x, B, dt_tok, A, chunk_size, initial_states=None, seq_idx=None):
    """h_t = [id_t == id_{t-1}] * exp(dt_t A_h) * h_{t-1} + dt_t * x_t (outer) B_t,  h_{-1} = init, id_{-1} = 0.

    dt_tok is the *activated* per-token step (b, L, H).  Returns, in fp64,
    out (b, C, H, P, N) with out[:, c] = h_{cQ-1} (out[:, 0] = init) and final = h_{L-1}.
    Nothing here knows about chunks except where the snapshots are taken."""
    batch, seqlen, nheads, headdim = x.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    ratio = nheads // ngroups
    nchunks = math.ceil(seqlen / chunk_size)
    h = (torch.zeros(batch, nheads, headdim, dstate, dtype=torch.float64) if initial_states is None
         else initial_states.double().clone())
    out = torch.empty(batch, nchunks, nheads, headdim, dstate, dtype=torch.float64)
    out[:, 0] = h
    xd, Bd, dtd, Ad = x.double(), B.double(), dt_tok.double(), A.double()
    prev = torch.zeros(batch, dtype=torch.long)
    for t in range(seqlen):
        a = torch.exp(dtd[:, t] * Ad[None, :])                       # (b,H)
        if seq_idx is not None:
            cur = seq_idx[:, t].long()
            a = a * (cur == prev)[:, None].double()
            prev = cur
        Bt = Bd[:, t].repeat_interleave(ratio, dim=1)                # (b,H,N)
        h = a[..., None, None] * h + dtd[:, t][..., None, None] * xd[:, t][..., None] * Bt[:, :, None, :]
        if (t + 1) % chunk_size == 0 and (t + 1) // chunk_size < nchunks:
            out[:, (t + 1) // chunk_size] = h
    return out, h


# --------------------------------------------------------------------------------------
# The callers on either side of the path inside a whole SSD forward (main.py:60-104): restated so that the
# library's kernels can be exercised in place, and pinned by a token-serial evaluation of y.
# --------------------------------------------------------------------------------------
def bmm_chunk_ref(a, b, chunk_size, seq_idx=None):
    """Follows kernels/ssd_bmm.py:46-87 (non-causal, grouped form).  a, b (batch, L, G, K) ->
    out (batch, C, G, Q, Q) fp32 with out[.., m, n] = sum_k a[cQ+m, g, k] * b[cQ+n, g, k]; rows / columns past the
    end of the sequence are zero; entries whose tokens belong to different sequences are zero."""
    batch, seqlen, ngroups, k = a.shape
    assert b.shape == a.shape
    nchunks = math.ceil(seqlen / chunk_size)
    pad = nchunks * chunk_size - seqlen
    af, bf = a.float(), b.float()
    if pad:
        af = F.pad(af, (0, 0, 0, 0, 0, pad))
        bf = F.pad(bf, (0, 0, 0, 0, 0, pad))
    af = af.reshape(batch, nchunks, chunk_size, ngroups, k)
    bf = bf.reshape(batch, nchunks, chunk_size, ngroups, k)
    out = torch.einsum("bcmgk,bcngk->bcgmn", af, bf)
    if seq_idx is not None:
        assert seq_idx.shape == (batch, seqlen)
        ids = seq_idx.long()
        # padded rows get -1 and padded columns -2, so they never match (:79-80)
        idm = F.pad(ids, (0, pad), value=-1).reshape(batch, nchunks, chunk_size)
        idn = F.pad(ids, (0, pad), value=-2).reshape(batch, nchunks, chunk_size)
        same = idm[:, :, :, None] == idn[:, :, None, :]
        out = out * same[:, :, None].float()
    return out


def chunk_scan_ref(cb, x, dt, dA_cumsum, C, states, D=None, z=None, seq_idx=None):
    """Follows kernels/ssd_chunk_scan.py:65-169 with IS_CAUSAL (the wrapper passes True, :213).
    y[cQ+m] = scale_m * (C[cQ+m] . states[c]) + sum_{k<=m} cb[m,k] * exp(min(dAcs_m - dAcs_k, 0)) * dt_k * x[cQ+k] + D x,
    scale_m = exp(dAcs_m) * [seq_idx[cQ+m] == seq_idx[cQ-1]] (the latter taken as 0 for the first chunk).
    Returns (out, out_x) in fp32: with z, out_x is y and out is y * z * sigmoid(z); without, (y, None)."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, Q = dt.shape
    _, _, ngroups, dstate = C.shape
    assert nheads % ngroups == 0
    assert cb.shape == (batch, nchunks, ngroups, Q, Q)
    assert states.shape == (batch, nchunks, nheads, headdim, dstate)
    ratio = nheads // ngroups
    pad = nchunks * Q - seqlen
    xf, Cf = x.float(), C.float()
    if pad:
        xf = F.pad(xf, (0, 0, 0, 0, 0, pad))
        Cf = F.pad(Cf, (0, 0, 0, 0, 0, pad))
    xc = xf.reshape(batch, nchunks, Q, nheads, headdim)
    Cc = Cf.reshape(batch, nchunks, Q, ngroups, dstate).repeat_interleave(ratio, dim=3)          # (b,c,Q,H,N)
    dacs = dA_cumsum.float().permute(0, 2, 1, 3)                                                 # (b,c,H,Q)
    dtc = dt.float().permute(0, 2, 1, 3)
    # contribution of the state entering the chunk (:94-117)
    scale = torch.exp(dacs)                                                                      # (b,c,H,Q)
    if seq_idx is not None:
        ids = F.pad(seq_idx.long(), (0, pad), value=-1).reshape(batch, nchunks, Q)
        prev = torch.zeros(batch, nchunks, dtype=torch.long)
        prev[:, 1:] = ids[:, :-1, -1]
        scale = scale * (ids == prev[:, :, None])[:, :, None, :].float()
    y = torch.einsum("bcmhn,bchpn->bcmhp", Cc, states.float()) * scale.permute(0, 1, 3, 2)[..., None]
    # intra-chunk part (:119-148)
    decay = torch.exp(torch.clamp(dacs[..., :, None] - dacs[..., None, :], max=0.0))            # (b,c,H,m,k)
    causal = torch.tril(torch.ones(Q, Q, dtype=torch.bool))
    cbh = cb.float().repeat_interleave(ratio, dim=2)                                             # (b,c,H,m,k)
    m = cbh * decay * dtc[..., None, :] * causal.float()
    y = y + torch.einsum("bchmk,bckhp->bcmhp", m, xc)
    if D is not None:
        Df = D.float()
        y = y + xc * (Df[None, None, None, :, :] if Df.dim() == 2 else Df[None, None, None, :, None])
    y = y.reshape(batch, nchunks * Q, nheads, headdim)[:, :seqlen]
    if z is None:
        return y, None
    zf = z.float()
    return y * zf * torch.sigmoid(zf), y


def chunk_scan_states_ref(C, states, dA_cumsum, seq_idx=None):
    """Follows kernels/ssd_chunk_scan.py:94-117 alone: the contribution of the state entering each chunk,
    y[b, cQ+m, h, :] = scale_m * (C[b, cQ+m, g, :] . states[b, c, h]),  scale_m = exp(dA_cumsum[b, h, c, m]) where
    seq_idx[b, cQ+m] == seq_idx[b, cQ-1] (taken as 0 for c == 0), else 0.  fp32 throughout: the reference's rounding
    of the states to C's element type (:110) is not restated.  Returns y (batch, seqlen, nheads, headdim) fp32."""
    batch, seqlen, ngroups, dstate = C.shape
    _, nchunks, nheads, headdim, _ = states.shape
    Q = dA_cumsum.shape[-1]
    ratio = nheads // ngroups
    y = torch.zeros(batch, seqlen, nheads, headdim, dtype=torch.float32)
    for c in range(nchunks):
        lo, hi = c * Q, min((c + 1) * Q, seqlen)
        Cc = C[:, lo:hi].float().repeat_interleave(ratio, dim=2)                      # (b, m, H, N)
        scale = torch.exp(dA_cumsum[:, :, c, :hi - lo].float()).permute(0, 2, 1)      # (b, m, H)
        if seq_idx is not None:
            prev = seq_idx[:, lo - 1].long() if c >= 1 else torch.zeros(batch, dtype=torch.long)
            scale = scale * (seq_idx[:, lo:hi].long() == prev[:, None]).float()[:, :, None]
        y[:, lo:hi] = torch.einsum("bmhn,bhpn->bmhp", Cc, states[:, c].float()) * scale[..., None]
    return y


def token_scan_ref(x, B, C, dt_tok, A, D=None, initial_states=None, seq_idx=None):
    """Token-serial selective scan in fp64, with no notion of chunks:
    h_t = [id_t == id_{t-1}] * exp(dt_t A_h) * h_{t-1} + dt_t * x_t (outer) B_t,  y_t = C_t . h_t + D x_t.
    Returns (y (b, L, H, P), h_{L-1})."""
    batch, seqlen, nheads, headdim = x.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    ratio = nheads // ngroups
    h = (torch.zeros(batch, nheads, headdim, dstate, dtype=torch.float64) if initial_states is None
         else initial_states.double().clone())
    xd, Bd, Cd, dtd, Ad = x.double(), B.double(), C.double(), dt_tok.double(), A.double()
    y = torch.empty(batch, seqlen, nheads, headdim, dtype=torch.float64)
    prev = torch.zeros(batch, dtype=torch.long)
    for t in range(seqlen):
        a = torch.exp(dtd[:, t] * Ad[None, :])
        if seq_idx is not None:
            cur = seq_idx[:, t].long()
            a = a * (cur == prev)[:, None].double()
            prev = cur
        Bt = Bd[:, t].repeat_interleave(ratio, dim=1)
        Ct = Cd[:, t].repeat_interleave(ratio, dim=1)
        h = a[..., None, None] * h + dtd[:, t][..., None, None] * xd[:, t][..., None] * Bt[:, :, None, :]
        y[:, t] = torch.einsum("bhpn,bhn->bhp", h, Ct)
        if D is not None:
            Dd = D.double()
            y[:, t] += xd[:, t] * (Dd[None] if Dd.dim() == 2 else Dd[None, :, None])
    return y, h


# --------------------------------------------------------------------------------------
# Seeded inputs for the five benchmark configurations
# --------------------------------------------------------------------------------------
CONFIGS = [
    dict(name="cfg0_cpu_fp32", b=1, L=1024, H=8, P=64, N=64, G=1, Q=256, dtype="fp32", init=False, nseq=0),
    dict(name="cfg1_mamba2_130m", b=8, L=2048, H=24, P=64, N=128, G=1, Q=256, dtype="bf16", init=False, nseq=0),
    dict(name="cfg2_mamba2_2p7b", b=4, L=8192, H=80, P=64, N=128, G=1, Q=256, dtype="bf16", init=True, nseq=0),
    dict(name="cfg3_varlen_packed", b=1, L=32768, H=80, P=64, N=128, G=1, Q=256, dtype="bf16", init=False, nseq=16),
    dict(name="cfg4_long_grouped", b=1, L=131072, H=128, P=64, N=128, G=8, Q=256, dtype="bf16", init=False, nseq=0),
]


def _softplus_inv(y):
    return y + torch.log(-torch.expm1(-y))


def make_inputs(cfg_index, **override):
    """Deterministic CPU inputs (generator seed 20240 + cfg_index).  ``override`` may shrink any dimension
    (b, L, H, P, N, G, Q, nseq, init, dtype) to make a CPU-sized case with the same value distributions.

    Returns a dict with the hot-path inputs x, B, dt, dA_cumsum (+ seq_idx, initial_states when the
    configuration has them) and the raw per-token quantities A, dt_tok used by the token-serial pin."""
    cfg = dict(CONFIGS[cfg_index])
    cfg.update(override)
    b, L, H, P, N, G, Q = (cfg[k] for k in "bLHPNGQ")
    dtype = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[cfg["dtype"]]
    g = torch.Generator().manual_seed(20240 + cfg_index)
    x = torch.randn(b, L, H, P, generator=g).to(dtype)
    Bm = torch.randn(b, L, G, N, generator=g).to(dtype)
    Cm = torch.randn(b, L, G, N, generator=g).to(dtype)   # drawn to keep the stream layout; unused by the path
    A = -torch.exp(torch.empty(H).uniform_(math.log(1.0), math.log(16.0), generator=g))
    dt_val = torch.exp(torch.empty(b, L, H).uniform_(math.log(1e-3), math.log(1e-1), generator=g))
    dt_bias = _softplus_inv(torch.full((H,), 1e-2))
    dt_raw = (_softplus_inv(dt_val) - dt_bias).to(dtype)
    dA_cumsum, dt = chunk_cumsum_ref(dt_raw, A, Q, dt_bias=dt_bias, dt_softplus=True)
    res = dict(cfg=cfg, x=x, B=Bm, C=Cm, A=A, dt=dt, dA_cumsum=dA_cumsum, dt_raw=dt_raw, dt_bias=dt_bias,
               seq_idx=None, initial_states=None)
    if cfg["init"]:
        res["initial_states"] = 0.1 * torch.randn(b, H, P, N, generator=g)
    if cfg["nseq"]:
        nseq = cfg["nseq"]
        raw = torch.empty(nseq).uniform_(512.0, 4096.0, generator=g)
        lens = torch.floor(raw * L / raw.sum()).long()
        lens[-1] += L - lens.sum()
        ids = torch.repeat_interleave(torch.arange(nseq), lens).to(torch.int32)
        res["seq_idx"] = ids.reshape(1, L).expand(b, L).contiguous()
        res["seq_lens"] = lens
    # activated per-token dt, (b, L, H), consistent with the (b,H,C,Q) tensor above
    C_ = dt.shape[2]
    res["dt_tok"] = dt.permute(0, 2, 3, 1).reshape(b, C_ * Q, H)[:, :L].contiguous()
    return res


def make_reference_inputs(n_groups=1, dstate=128, nheads=80, headdim=64, seq_len=2048, dtype=torch.bfloat16,
                          chunk_size=256, batch_size=1, seed=42):
    """The reference's own test case (kernels/rand_data.py:4-25; main.py:166-179 runs it with dt_softplus=False,
    dt_bias, no initial states, no seq_idx, out_dtype = C.dtype = bf16).  Returns x, A, B, C, D, dt, dt_bias in the
    reference's order, on the CPU."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((batch_size, seq_len, nheads, headdim), generator=g).to(dtype)
    A = (torch.rand((nheads,), generator=g) * -1).to(dtype)                       # can be 0: no decay at all
    B = torch.randn((batch_size, seq_len, n_groups, dstate), generator=g).to(dtype)
    C = torch.randn((batch_size, seq_len, n_groups, dstate), generator=g).to(dtype)
    D = torch.randn((nheads,), generator=g).to(dtype)
    dt = (torch.rand((batch_size, seq_len, nheads), generator=g) * 0.5 + 0.5).to(dtype)
    dt_bias = (torch.rand((nheads,), generator=g) * 0.5 - 0.25).to(dtype)
    return x, A, B, C, D, dt, dt_bias


def algorithmic_bytes(cfg, with_states=False):
    """Bytes every input and contract output is counted once (out in fp32); the per-chunk states tensor is an
    intermediate and is only counted when ``with_states``."""
    b, L, H, P, N, G, Q = (cfg[k] for k in "bLHPNGQ")
    C = math.ceil(L / Q)
    esz = 4 if cfg["dtype"] == "fp32" else 2
    n = b * L * H * P * esz + b * L * G * N * esz + 2 * b * H * C * Q * 4
    if cfg.get("nseq"):
        n += b * L * 4
    if cfg.get("init"):
        n += b * H * P * N * 4
    S = b * C * H * P * N * 4
    n += S + b * H * P * N * 4
    if with_states:
        n += S
    return n


def algorithmic_flops(cfg):
    b, L, H, P, N, Q = (cfg[k] for k in "bLHPNQ")
    C = math.ceil(L / Q)
    return 2 * b * L * H * P * N + 2 * b * C * H * P * N
