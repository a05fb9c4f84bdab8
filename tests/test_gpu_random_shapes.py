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
