"""GPU parity of the ticket / flag-chain kernel (ssd_fused_chunk_state_passing_fwd_ws), forced through the C ABI in
each of its variants, against the CPU oracle on the same seeded inputs.

The kernel replaces the reference's global barrier (kernels/fused_globalbar.py:130-137) and its completion counters
and throttle semaphore (kernels/fused_concurrent.py:81-84, 141, 205-208); the reference has no test of either beyond
main.py:164-190.  Tolerance: rtol 2e-3 / atol 1e-3 against the fp32 oracle (bf16 inputs, fp32 states)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-3, 1e-3
LOCAL, GLOBAL = 2, 3            # SSD_KERNEL_CHAIN_LOCAL / SSD_KERNEL_CHAIN_GLOBAL


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


def _chain_case(ops, oracle, d, kernel, r, name, clamp=True, spin_limit=0):
    x, B, dt, dAcs, seq, init = d["x"], d["B"], d["dt"], d["dA_cumsum"], d["seq_idx"], d["initial_states"]
    want_out, want_fin = oracle.fused_ref(B, x, dt, dAcs, initial_states=init, seq_idx=seq, clamp=clamp)
    ws = torch.full((max(1 << 16, 64 + x.shape[0] * x.shape[2] * (x.shape[3] // 32) * dt.shape[2]),), -1,
                    dtype=torch.int32, device="cuda")           # garbage on purpose: the call clears what it uses
    print(f"[{name}] kernel={kernel} chunks/item={r} x{tuple(x.shape)} seq={seq is not None} init={init is not None}", flush=True)
    out, fin = ops._fused_chunk_state_state_passing_fwd(
        _dev(B), _dev(x), _dev(dt), _dev(dAcs), torch.float32, initial_states=_dev(init), seq_idx=_dev(seq),
        _clamp=clamp, _kernel=kernel, _chunks_per_item=r, _workspace=ws, _spin_limit=spin_limit)
    status = ops._fused_workspace_status(ws)
    assert status == 0, f"{name}: workspace status {status}"
    for what, got, want in (("out", out, want_out), ("final", fin, want_fin)):
        bad, worst = _mismatches(got, want)
        print(f"[{name}.{what}] max_abs={worst:.3e} mismatches={bad}/{want.numel()}", flush=True)
        assert bad == 0, f"{name}.{what}: {bad} mismatches, max abs err {worst:.3e}"
    return out, fin


SHAPES = [
    dict(b=2, L=2048, H=8, init=True),                   # 8 chunks, initial states
    dict(L=2000, H=8, nseq=5, init=True),                # ragged last chunk, packed sequences, initial states
    dict(L=2304, H=8),                                   # 9 chunks: items of 2 or 4 chunks do not divide them
    dict(Q=128, L=1408, N=64, H=8),                      # chunk 128 (four steps, ring of four), dstate 64
    dict(P=128, H=4, G=2, L=1280),                       # headdim 128, grouped B
    dict(P=96, H=4, L=1024),                             # three row slices per head: tiles of a unit straddle heads
    dict(L=1, H=8),                                      # a single token
    dict(L=257, H=8),                                    # one full chunk and one token
    dict(b=1, L=8192, H=16, nseq=3),                     # 32 chunks on few units: every workgroup waits on the chain
]


@pytest.mark.parametrize("r", [1, 2, 4])
@pytest.mark.parametrize("kernel", [LOCAL, GLOBAL], ids=["local", "global"])
@pytest.mark.parametrize("kw", SHAPES, ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))
def test_chain_kernel_variants(ops, oracle, kw, kernel, r):
    base = dict(b=2, L=1024, H=6, G=1)
    base.update(kw)
    _chain_case(ops, oracle, oracle.make_inputs(1, **base), kernel, r, f"chain.k{kernel}.r{r}")


def _bf16_workspace_ints(x, B, dt, r):
    # header + a flag per (state tile, chunk), rounded up to 256 bytes, then 32 x dstate fp32 per (state tile, item)
    tiles, C, N = x.shape[0] * x.shape[2] * (x.shape[3] // 32), dt.shape[2], B.shape[-1]
    return (128 + tiles * C + 63) // 64 * 64 + tiles * ((C + r - 1) // r) * 32 * N


@pytest.mark.parametrize("r", [2, 4])
@pytest.mark.parametrize("kernel", [LOCAL, GLOBAL], ids=["local", "global"])
@pytest.mark.parametrize("kw", SHAPES + [dict(L=4096, H=8, nseq=6, init=True)], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))
def test_chain_bf16_passed_states(ops, oracle, kw, kernel, r):
    # bf16 `out` (what the reference's main.py asks for, out_dtype = C.dtype): the state that crosses between work
    # items stays fp32 (kernels/ssd_state_passing.py:61-84 keeps it in registers), through a slot of the workspace.  So
    # the final states are those of the fp32 call bit for bit, and `out` is the fp32 call's `out` rounded once.
    from ssd_amd import _lib
    base = dict(b=2, L=1024, H=6, G=1)
    base.update(kw)
    d = oracle.make_inputs(1, **base)
    name = f"chain.bf16out.k{kernel}.r{r}"
    out32, fin32 = _chain_case(ops, oracle, d, kernel, r, name + ".fp32")
    x, B, dt, dAcs, seq, init = d["x"], d["B"], d["dt"], d["dA_cumsum"], d["seq_idx"], d["initial_states"]
    n_ints = _bf16_workspace_ints(x, B, dt, r)
    dims = _lib.dims_arg(x.shape[0], x.shape[1], x.shape[2], x.shape[3], B.shape[-1], B.shape[2], dt.shape[3], dt.shape[2])
    assert int(_lib.load().ssd_fused_workspace_bytes_for(dims, _lib.SSD_BF16, r)) == 4 * n_ints
    ws = torch.full((n_ints,), -1, dtype=torch.int32, device="cuda")           # garbage, the fp32 slots included
    print(f"[{name}] x{tuple(x.shape)} workspace {4 * n_ints} bytes", flush=True)
    out16, fin16 = ops._fused_chunk_state_state_passing_fwd(
        _dev(B), _dev(x), _dev(dt), _dev(dAcs), torch.bfloat16, initial_states=_dev(init), seq_idx=_dev(seq),
        _kernel=kernel, _chunks_per_item=r, _workspace=ws)
    assert ops._fused_workspace_status(ws) == 0
    assert out16.dtype == torch.bfloat16 and torch.isfinite(out16.float()).all()
    assert torch.equal(fin16, fin32), f"{name}: final states differ, max {float((fin16 - fin32).abs().max()):.3e}"
    assert torch.equal(out16, out32.to(torch.bfloat16)), f"{name}: out differs, max {float((out16.float() - out32).abs().max()):.3e}"


def test_chain_bf16_passed_states_left_to_the_library(ops, oracle):
    # no hooks: the wrapper sizes its own workspace for bf16 `out` and the library picks the kernel (32 chunks on 40
    # units: the chain kernel); a second call reuses the workspace with the next epoch
    d = oracle.make_inputs(2, b=1, L=8192, H=40)
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    for i in range(2):
        out, fin = ops._fused_chunk_state_state_passing_fwd(*args, torch.bfloat16, initial_states=_dev(d["initial_states"]))
        torch.cuda.synchronize()
        assert out.dtype == torch.bfloat16
        bad, worst = _mismatches(out, want_out, rtol=RTOL + 2.0 ** -8)
        assert bad == 0, f"call {i}: out {bad} mismatches, max {worst:.3e}"
        bad, worst = _mismatches(fin, want_fin)
        assert bad == 0, f"call {i}: final {bad} mismatches, max {worst:.3e}"


@pytest.mark.parametrize("r", [2, 4])
@pytest.mark.parametrize("kernel", [LOCAL, GLOBAL], ids=["local", "global"])
def test_chain_items_cut_by_sequence_starts(ops, oracle, kernel, r):
    # Sequence starts placed at every position inside a work item: in chunk 1 (mid-chunk), in chunks 6 and 7 (two in one
    # item, one of them on a chunk's first token), in chunk 11 (the item's last chunk) and none in the last item.  The
    # states behind the last start of an item are handed on before the item has seen its predecessor's state.
    d = oracle.make_inputs(1, b=2, L=4096, H=8, init=True)
    starts = [256 + 100, 6 * 256, 7 * 256 + 255, 11 * 256 + 17]
    ids = torch.zeros(4096, dtype=torch.int32)
    for s0 in starts:
        ids[s0:] += 1
    d["seq_idx"] = ids.reshape(1, -1).expand(2, -1).contiguous()
    _chain_case(ops, oracle, d, kernel, r, f"chain.cut.k{kernel}.r{r}")


@pytest.mark.timeout(600)
@pytest.mark.parametrize("cfg", [2, 3], ids=["cfg2", "cfg3"])
def test_chain_kernel_at_benchmark_configs(ops, oracle, cfg):
    # what the library picks for these two by itself (cfg 4 is compared slice-wise in test_gpu_parity.py)
    d = oracle.make_inputs(cfg)
    _chain_case(ops, oracle, d, 1, 0, f"chain.cfg{cfg}")


@pytest.mark.parametrize("kw, family, r", [
    (dict(b=1, L=8192, H=80), "chain", 2),        # 40 units x 32 chunks: two chunks per item fill the device evenly
    (dict(b=8, L=2048, H=80), "chain", 2),        # 8 chunks only, 320 units
    (dict(b=3, L=4096, H=80), "chain", 4),
    (dict(b=4, L=2048, H=80), "four_tile", 0),    # 160 units x 8 chunks: one workgroup per unit is faster
    (dict(b=2, L=2048, H=80), "token_split", 0),  # 80 units x 8 chunks
], ids=["b1-L8192", "b8-L2048", "b3-L4096", "b4-L2048", "b2-L2048"])
def test_shapes_between_the_benchmark_configs_on_the_kernel_the_library_picks(ops, oracle, kw, family, r):
    # the choice is made from an estimate of each family's duration; whatever it picks has to be right
    d = oracle.make_inputs(2, **kw)
    cfg = d["cfg"]
    plan = ops.fused_plan(cfg["b"], cfg["L"], cfg["H"], cfg["P"], cfg["N"], cfg["G"], cfg["Q"])
    assert (plan["family"], plan["chunks_per_item"]) == (family, r), plan
    _chain_case(ops, oracle, d, 0, 0, "auto." + "-".join(f"{k}{v}" for k, v in kw.items()))


@pytest.mark.parametrize("kernel", [0, LOCAL, GLOBAL], ids=["auto", "local", "global"])
@pytest.mark.parametrize("kw", [dict(b=2, L=2048, H=8, init=True), dict(L=2000, H=8, nseq=5, init=True),
                                dict(Q=128, L=1408, N=64, H=8)], ids=["base", "ragged-seq", "q128-n64"])
def test_dt_preparation_and_chain_kernel_in_one_call(ops, oracle, kw, kernel):
    # kernels/ssd_chunk_state.py:176-199 followed by the fused call, as one call with a workspace: the producer's launch
    # clears the chain kernel's workspace (garbage here) on its way; same bits as the two calls made separately
    d = oracle.make_inputs(2, **kw)
    Q = d["cfg"]["Q"]
    raw, A, bias, seq, init = d["dt_raw"], d["A"], d["dt_bias"], d["seq_idx"], d["initial_states"]
    want_da, want_dt = oracle.chunk_cumsum_ref(raw, A, Q, dt_bias=bias, dt_softplus=True)
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], want_dt, want_da, initial_states=init, seq_idx=seq)
    for rep in range(2):                                   # the second call finds the workspace as the first left it
        ws = torch.full((1 << 16,), -1, dtype=torch.int32, device="cuda") if rep == 0 else ws
        out, fin, dA, dt = ops._fused_cumsum_chunk_state_state_passing_fwd(
            _dev(d["B"]), _dev(d["x"]), _dev(raw), _dev(A), Q, torch.float32, dt_bias=_dev(bias), dt_softplus=True,
            initial_states=_dev(init), seq_idx=_dev(seq), _kernel=kernel, _workspace=ws)
        assert ops._fused_workspace_status(ws) == 0
        for what, got, want, rtol, atol in (("dt", dt, want_dt, 2e-6, 1e-9), ("dA_cumsum", dA, want_da, 1e-5, 1e-6),
                                            ("out", out, want_out, RTOL, ATOL), ("final", fin, want_fin, RTOL, ATOL)):
            bad, worst = _mismatches(got, want, rtol, atol)
            assert bad == 0, f"prep+chain.{what}: {bad} mismatches, max abs err {worst:.3e}"
        dA2, dt2 = ops._chunk_cumsum_fwd(_dev(raw), _dev(A), Q, dt_bias=_dev(bias), dt_softplus=True)
        out2, fin2 = ops._fused_chunk_state_state_passing_fwd(_dev(d["B"]), _dev(d["x"]), dt2, dA2, torch.float32,
                                                              initial_states=_dev(init), seq_idx=_dev(seq), _kernel=kernel,
                                                              _workspace=torch.full((1 << 16,), -1, dtype=torch.int32, device="cuda"))
        torch.cuda.synchronize()
        assert torch.equal(dt2, dt) and torch.equal(dA2, dA) and torch.equal(out2, out) and torch.equal(fin2, fin)
    # the same call with bf16 passed states on the wrapper's own workspace: final states as above, `out` rounded once
    out16, fin16, _, _ = ops._fused_cumsum_chunk_state_state_passing_fwd(
        _dev(d["B"]), _dev(d["x"]), _dev(raw), _dev(A), Q, torch.bfloat16, dt_bias=_dev(bias), dt_softplus=True,
        initial_states=_dev(init), seq_idx=_dev(seq), _kernel=kernel)
    torch.cuda.synchronize()
    assert out16.dtype == torch.bfloat16
    if kernel != 0:                                        # same kernel, same chunks per item unless the library chose
        bad, worst = _mismatches(fin16, fin.cpu(), 1e-5, 1e-6)
        assert bad == 0, f"prep+chain.bf16.final: {bad} mismatches, max abs err {worst:.3e}"
    bad, worst = _mismatches(out16, want_out, RTOL + 2.0 ** -8, ATOL)
    assert bad == 0, f"prep+chain.bf16.out: {bad} mismatches, max abs err {worst:.3e}"
    bad, worst = _mismatches(fin16, want_fin)
    assert bad == 0, f"prep+chain.bf16.final: {bad} mismatches, max abs err {worst:.3e}"


def test_chain_local_with_fewer_units_than_xcds(ops, oracle):
    # One unit (two heads), per-XCD tickets insisted on: the unit belongs to one XCD, and that XCD must get a workgroup
    # whichever XCD the launch happens to start its round of workgroups on -- small launches in front move that turn.
    # (A launch of as many workgroups as work items, two here, once left the unit's XCD without one: every output
    # wrong and no error reported.)
    d = oracle.make_inputs(2, b=1, L=1730, H=2, init=True)
    for i in range(12):
        for _ in range(i):
            torch.zeros(64 * (i + 1), device="cuda")          # a one-workgroup launch each
        _chain_case(ops, oracle, d, LOCAL, 4, f"chain.local.one_unit[{i}]")


def test_chain_matches_the_other_fused_kernels(ops, oracle):
    # same inputs through the chain kernel and through the kernel the workspace-less entry point picks
    d = oracle.make_inputs(2, b=2, L=4096, H=16)
    out, fin = _chain_case(ops, oracle, d, LOCAL, 4, "chain.vs")
    lib = __import__("ssd_amd")._lib
    xd, Bd, dtd, dAd, initd = map(_dev, (d["x"], d["B"], d["dt"], d["dA_cumsum"], d["initial_states"]))
    old = ops.set_token_split(1)       # keeps the library from picking the chain kernel
    try:
        out2, fin2 = ops._fused_chunk_state_state_passing_fwd(Bd, xd, dtd, dAd, torch.float32, initial_states=initd)
        torch.cuda.synchronize()
    finally:
        ops.set_token_split(old)
    assert float((out - out2).abs().max()) <= 1e-4 and float((fin - fin2).abs().max()) <= 1e-4
    assert lib is not None


def test_chain_without_the_clamp(ops, oracle):
    # clamp = 0 is what the reference's fused kernels compute (fused_globalbar.py:106); it differs from the clamped
    # form only where dA_cumsum is not monotone
    d = oracle.make_inputs(1, b=2, L=2048, H=8)
    g = torch.Generator().manual_seed(5)
    d["dA_cumsum"] = d["dA_cumsum"] + 0.3 * torch.randn(d["dA_cumsum"].shape, generator=g)
    a = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], clamp=True)[0]
    b = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], clamp=False)[0]
    assert float((a - b).abs().max()) > 1e-2            # the two semantics do differ on these inputs
    for clamp in (True, False):
        _chain_case(ops, oracle, d, LOCAL, 4, f"chain.clamp{int(clamp)}", clamp=clamp)


def test_chain_bounded_wait_gives_up_and_reports(ops, oracle):
    # Four units, 32 chunks each, one poll allowed: waves reach their chain step long before their predecessors
    # have finished, give up, and say so.  The launch still drains (every wave raises its flag), and the next call
    # on the same workspace is clean.
    d = oracle.make_inputs(1, b=1, L=8192, H=8)
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    ws = torch.zeros(1 << 16, dtype=torch.int32, device="cuda")
    ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, _kernel=GLOBAL, _chunks_per_item=1, _workspace=ws,
                                             _spin_limit=1)
    assert ops._fused_workspace_status(ws) == -7        # SSD_ERR_CHAIN_TIMEOUT
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"])
    out, fin = ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, _kernel=GLOBAL, _chunks_per_item=1,
                                                        _workspace=ws)
    assert ops._fused_workspace_status(ws) == 0
    assert _mismatches(out, want_out)[0] == 0 and _mismatches(fin, want_fin)[0] == 0


def test_chain_rejections(ops, oracle):
    from ssd_amd import _lib
    d = oracle.make_inputs(1, b=2, L=1024, H=8)
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    small = torch.zeros(8, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="workspace"):                       # forced, workspace too small
        ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, _kernel=1, _workspace=small)
    with pytest.raises(RuntimeError, match="workspace"):                       # forced, fp16 out is not its job
        ops._fused_chunk_state_state_passing_fwd(*args, torch.float16, _kernel=1)
    with pytest.raises(RuntimeError, match="workspace"):                       # forced, bf16 out with items of one chunk
        ops._fused_chunk_state_state_passing_fwd(*args, torch.bfloat16, _kernel=1, _chunks_per_item=1)
    flags_only = torch.zeros(1 << 16, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="workspace"):                       # forced, bf16 out, no room for the fp32 copies
        ops._fused_chunk_state_state_passing_fwd(*args, torch.bfloat16, _kernel=1, _workspace=flags_only)
    out16, _ = ops._fused_chunk_state_state_passing_fwd(*args, torch.bfloat16, _workspace=flags_only)      # not forced: another kernel
    assert out16.dtype == torch.bfloat16
    # left to itself the library falls back to its other kernels in both situations
    out, fin = ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, _workspace=small)
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"])
    torch.cuda.synchronize()
    assert _mismatches(out, want_out)[0] == 0 and _mismatches(fin, want_fin)[0] == 0
    assert _lib.SSD_ERR_SCRATCH == -6


def test_chain_back_to_back_and_other_stream(ops, oracle):
    # the workspace is cleared by every call: launches back to back on one stream reuse it
    d = oracle.make_inputs(2, b=1, L=4096, H=16)
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    initd = _dev(d["initial_states"])
    ws = torch.empty(1 << 16, dtype=torch.int32, device="cuda")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        results = [ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, initial_states=initd, _kernel=LOCAL,
                                                            _workspace=ws) for _ in range(4)]
        assert ops._fused_workspace_status(ws) == 0
    stream.synchronize()
    for out, fin in results[1:]:
        assert torch.equal(out, results[0][0]) and torch.equal(fin, results[0][1])
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
    assert _mismatches(results[0][0], want_out)[0] == 0 and _mismatches(results[0][1], want_fin)[0] == 0


@pytest.mark.parametrize("kernel", [LOCAL, GLOBAL], ids=["local", "global"])
def test_chain_launches_competing_for_the_compute_units(ops, oracle, kernel):
    # Two streams, each with chain launches that want every compute unit for themselves (one workgroup fills a compute
    # unit: registers and LDS), a workspace each: workgroups of one launch start as those of the other leave, so neither
    # launch has all its workgroups resident -- the case the ticket order is for (an item only waits for smaller
    # tickets, and tickets are drawn by running workgroups).  Every result must be right and no wait may run out.
    d = oracle.make_inputs(2, b=2, L=8192, H=40)
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    initd = _dev(d["initial_states"])
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    spaces = [torch.empty(1 << 18, dtype=torch.int32, device="cuda") for _ in streams]
    results = [[], []]
    torch.cuda.synchronize()
    for rep in range(4):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                results[i].append(ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, initial_states=initd,
                                                                           _kernel=kernel, _workspace=spaces[i]))
    torch.cuda.synchronize()
    for i, st in enumerate(streams):
        assert ops._fused_workspace_status(spaces[i]) == 0
        for out, fin in results[i]:
            assert _mismatches(out, want_out)[0] == 0 and _mismatches(fin, want_fin)[0] == 0


def test_chain_workspace_kept_across_calls_with_epochs(ops, oracle):
    # ssd_fused_opts.epoch: a workspace that only these calls touch, cleared once (epoch 0) and from then on told its
    # epoch (2, 3, ...): no fill launch, flags carry the epoch, ticket counters alternate between two banks.  Shapes,
    # chunks per item and the way states cross compute units change from call to call; every call against the oracle.
    cases = [(dict(b=2, L=2048, H=8, init=True), LOCAL, 4), (dict(L=2000, H=8, nseq=5, init=True), GLOBAL, 2),
             (dict(L=2304, H=8), LOCAL, 1), (dict(b=1, L=4096, H=16), GLOBAL, 4), (dict(b=2, L=2048, H=8, init=True), LOCAL, 2),
             (dict(P=128, H=4, G=2, L=1280), LOCAL, 4), (dict(b=1, L=4096, H=16), LOCAL, 4), (dict(L=2304, H=8), GLOBAL, 4)]
    ws = torch.full((1 << 16,), -1, dtype=torch.int32, device="cuda")
    epoch, cleared = 0, 0
    for i, (kw, kernel, r) in enumerate(cases * 2):
        d = oracle.make_inputs(3 if "nseq" in kw else 2, **kw)
        want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"],
                                              seq_idx=d["seq_idx"])
        # the promise of an epoch covers the flags the last clearing covered: a call with more (state tile, chunk) pairs
        # starts over with epoch 0 (twice in this sequence)
        pairs = d["x"].shape[0] * d["x"].shape[2] * (d["x"].shape[3] // 32) * d["dt"].shape[2]
        if pairs > cleared:
            epoch, cleared = 0, pairs
        print(f"[epochs {i}] {kw} kernel={kernel} chunks/item={r} epoch={epoch} pairs={pairs}", flush=True)
        out, fin = ops._fused_chunk_state_state_passing_fwd(
            *[_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")], torch.float32, initial_states=_dev(d["initial_states"]),
            seq_idx=_dev(d["seq_idx"]), _kernel=kernel, _chunks_per_item=r, _workspace=ws, _epoch=epoch)
        assert ops._fused_workspace_status(ws) == 0
        assert _mismatches(out, want_out)[0] == 0 and _mismatches(fin, want_fin)[0] == 0, (i, kw)
        epoch = 2 if epoch == 0 else epoch + 1
    # a wait that runs out is reported for its own launch only, and the epochs go on
    d = oracle.make_inputs(2, b=1, L=4096, H=16)
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, _kernel=GLOBAL, _chunks_per_item=1, _workspace=ws,
                                             _epoch=epoch, _spin_limit=1)
    assert ops._fused_workspace_status(ws) == -7
    out, fin = ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, _kernel=GLOBAL, _chunks_per_item=1, _workspace=ws,
                                                        _epoch=epoch + 1)
    assert ops._fused_workspace_status(ws) == 0
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"])
    assert _mismatches(out, want_out)[0] == 0 and _mismatches(fin, want_fin)[0] == 0


def test_wrapper_keeps_its_own_workspace(ops, oracle):
    # without a workspace argument the wrapper uses one of its own per (device, stream) and advances its epoch only when
    # the chain kernel served the call: shapes that go to other kernel families in between must not disturb it
    shapes = [dict(b=1, L=8192, H=80), dict(b=2, L=2048, H=8), dict(b=4, L=2048, H=80), dict(b=1, L=8192, H=80),
              dict(b=3, L=4096, H=80), dict(b=2, L=2048, H=80), dict(b=1, L=8192, H=80)]
    wants = {}
    for rep in range(2):
        for i, kw in enumerate(shapes):
            d = oracle.make_inputs(2, **kw)
            key = str(kw)
            if key not in wants:
                wants[key] = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
            out, fin = ops._fused_chunk_state_state_passing_fwd(*[_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")], torch.float32,
                                                                initial_states=_dev(d["initial_states"]))
            torch.cuda.synchronize()
            assert _mismatches(out, wants[key][0])[0] == 0 and _mismatches(fin, wants[key][1])[0] == 0, (rep, i, kw)
    # and on a second stream, with a workspace of its own
    st = torch.cuda.Stream()
    st.wait_stream(torch.cuda.current_stream())
    d = oracle.make_inputs(2, b=1, L=8192, H=80)
    with torch.cuda.stream(st):
        for _ in range(3):
            out, fin = ops._fused_chunk_state_state_passing_fwd(*[_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")], torch.float32,
                                                                initial_states=_dev(d["initial_states"]))
    st.synchronize()
    key = str(dict(b=1, L=8192, H=80))
    assert _mismatches(out, wants[key][0])[0] == 0 and _mismatches(fin, wants[key][1])[0] == 0


def test_chain_reports_a_workspace_that_is_not_what_the_epoch_promises(ops, oracle):
    """ssd_fused_opts.epoch > 0 promises that the launch before was epoch - 1 and that the call looks at no more flags
    than the last clearing covered.  A small call clears 256 flags; a larger one with epoch 2 looks at 512, and the
    memory behind the cleared part holds the value 2 -- every wait would be skipped.  The kernel notices at ticket 0 and
    ssd_fused_workspace_status says so (SSD_ERR_CHAIN_WORKSPACE); an epoch that does not follow the one before is
    reported too.  The wrappers' own workspace is not exposed to this: they clear again when a call needs more."""
    from ssd_amd import ops as ops_module
    small = oracle.make_inputs(2, b=2, L=2048, H=8)            # 32 state tiles x 8 chunks
    big = oracle.make_inputs(2, b=1, L=4096, H=16)             # 32 x 16
    want = oracle.fused_ref(big["B"], big["x"], big["dt"], big["dA_cumsum"], initial_states=big["initial_states"])
    run = lambda d, **kw: ops._fused_chunk_state_state_passing_fwd(
        *[_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")], torch.float32, initial_states=_dev(d["initial_states"]), **kw)
    ws = torch.full((1 << 16,), 2, dtype=torch.int32, device="cuda")
    run(small, _kernel=GLOBAL, _workspace=ws, _epoch=0)
    assert ops._fused_workspace_status(ws) == 0
    print("[promise] more flags than were cleared, epoch 2", flush=True)
    run(big, _kernel=GLOBAL, _workspace=ws, _epoch=2, _spin_limit=64)
    assert ops._fused_workspace_status(ws) == -10
    # started over, the same call is clean
    out, fin = run(big, _kernel=GLOBAL, _workspace=ws, _epoch=0)
    assert ops._fused_workspace_status(ws) == 0
    assert _mismatches(out, want[0])[0] == 0 and _mismatches(fin, want[1])[0] == 0
    print("[promise] epoch 4 behind epoch 1, epoch 5 behind epoch 1", flush=True)
    run(big, _kernel=GLOBAL, _workspace=ws, _epoch=4, _spin_limit=64)       # parity of a launch nobody made: its counters are zero
    assert ops._fused_workspace_status(ws) == -10
    run(big, _kernel=GLOBAL, _workspace=ws, _epoch=0)
    run(big, _kernel=GLOBAL, _workspace=ws, _epoch=3, _spin_limit=64)       # same parity as epoch 1: its counters are used up
    assert ops._fused_workspace_status(ws) == -10
    # the wrappers' own workspace: small call, then the memory behind its flags poisoned with the next epoch, then the
    # larger call -- which must clear again by itself
    ops.release_workspaces()
    run(small, _kernel=GLOBAL)
    assert ops.fused_status() == 0
    (kept,) = [k for key, k in ops_module._WORKSPACES.items() if key[0] == torch.cuda.current_device()]
    kept.tensor[128 + 256:].fill_(2)
    out, fin = run(big, _kernel=GLOBAL)
    assert ops.fused_status() == 0
    assert _mismatches(out, want[0])[0] == 0 and _mismatches(fin, want[1])[0] == 0
    out, fin = run(big, _kernel=GLOBAL)                         # and goes on with epochs from there
    assert ops.fused_status() == 0 and kept.epochs.last == 2
    assert _mismatches(out, want[0])[0] == 0 and _mismatches(fin, want[1])[0] == 0


def test_chain_failures_reach_the_caller_of_the_plain_wrappers(ops, oracle):
    """The drop-in wrappers keep their workspace to themselves; fused_status() is how their caller learns that the last
    launch failed.  One poll allowed: waves give up (and still raise their flags, so the launch drains) -> -7; the next
    call is clean."""
    d = oracle.make_inputs(1, b=1, L=8192, H=8)
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    ops.release_workspaces()
    assert ops.fused_status() == 0                              # nothing kept yet
    ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, _kernel=GLOBAL, _chunks_per_item=1, _spin_limit=1)
    assert ops.fused_status() == -7
    out, fin = ops._fused_chunk_state_state_passing_fwd_concurrent(*args, torch.float32)
    assert ops.fused_status() == 0
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"])
    assert _mismatches(out, want_out)[0] == 0 and _mismatches(fin, want_fin)[0] == 0


def test_chain_reports_xcds_that_are_not_what_it_assumed(ops, oracle):
    """LOCAL deals the units to one ticket counter per XCD and relies on a workgroup of every XCD showing up.  With the
    test hook the library is told a wrong number of XCDs: 4 makes pairs of XCDs share a counter (SSD_ERR_CHAIN_XCD), 16
    leaves half of the counters without any workgroup, so their units are never computed (SSD_ERR_CHAIN_INCOMPLETE --
    no error bit is set by anybody, the ticket counters tell).  Waits are short, every kernel exits normally."""
    d = oracle.make_inputs(2, b=2, L=4096, H=16)                # 16 units x 16 chunks
    args = [_dev(d[k]) for k in ("B", "x", "dt", "dA_cumsum")]
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
    ws = torch.zeros(1 << 16, dtype=torch.int32, device="cuda")
    run = lambda **kw: ops._fused_chunk_state_state_passing_fwd(*args, torch.float32, initial_states=_dev(d["initial_states"]),
                                                                _kernel=LOCAL, _chunks_per_item=2, _workspace=ws, **kw)
    try:
        for xcds, code in ((4, -8), (16, -9)):
            print(f"[xcds] told {xcds}", flush=True)
            assert ops.set_chain_xcds(xcds) in (0, 4)
            run(_spin_limit=16)
            assert ops._fused_workspace_status(ws) == code
    finally:
        ops.set_chain_xcds(0)
    out, fin = run()
    assert ops._fused_workspace_status(ws) == 0
    assert _mismatches(out, want_out)[0] == 0 and _mismatches(fin, want_fin)[0] == 0


def test_chain_with_an_out_view_that_shares_cache_lines_between_tiles(ops, oracle):
    """The per-XCD variant reads passed states back with plain loads, which is only safe while no two state tiles share
    a 128-byte line.  A C-ABI caller may hand over an `out` that starts 16 bytes into an allocation: the call must still
    be right (the library then exchanges the states through memory, whatever variant was asked for)."""
    import ctypes
    from ssd_amd import _lib
    lib = _lib.load()
    d = oracle.make_inputs(2, b=2, L=2048, H=32)                # 32 units: the library's own choice is the per-XCD variant
    want_out, want_fin = oracle.fused_ref(d["B"], d["x"], d["dt"], d["dA_cumsum"], initial_states=d["initial_states"])
    x, B, dt, dA, init = (_dev(d[k]) for k in ("x", "B", "dt", "dA_cumsum", "initial_states"))
    b, L, H, P = x.shape
    C, Q, N = dt.shape[2], dt.shape[3], B.shape[-1]
    dims = _lib.dims_arg(b, L, H, P, N, 1, Q, C)
    ws = torch.full((1 << 16,), -1, dtype=torch.int32, device="cuda")
    for kernel in (LOCAL, 1):
        buf = torch.full((b * C * H * P * N + 4,), float("nan"), device="cuda")
        out = buf[4:].view(b, C, H, P, N)
        assert out.data_ptr() % 128 == 16
        fin = torch.full((b, H, P, N), float("nan"), device="cuda")
        used = ctypes.c_int32(0)
        opts = _lib.SsdFusedOpts(ws.data_ptr(), ws.numel() * 4, 0, kernel, 0, 0, ctypes.pointer(used))
        T = _lib.tensor_arg
        print(f"[out view] kernel={kernel}", flush=True)
        rc = lib.ssd_fused_chunk_state_passing_fwd_ws(T(x), T(B), T(dt), T(dA), T(None), T(init), T(None), T(out), T(fin), dims, 1,
                                                      ctypes.byref(opts), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0 and used.value == 1
        assert ops._fused_workspace_status(ws) == 0
        assert _mismatches(out, want_out)[0] == 0 and _mismatches(fin, want_fin)[0] == 0


@pytest.mark.parametrize("kw", [dict(b=2, L=2048, H=8), dict(L=2000, H=8), dict(Q=128, L=1408, N=64, H=8), dict(P=128, H=4, G=2, L=1280)],
                         ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))
def test_traffic_floor_kernel_covers_every_output_tile(ops, oracle, kw):
    """ssd_measure_traffic_floor moves the fused call's bytes and computes nothing; bench.py prices the fused kernels
    against its duration.  What can be checked of it: it writes every element of `out` (here NaN before, zero after --
    a tile it skipped would make the floor too low) and touches nothing else."""
    base = dict(b=2, L=1024, H=6, G=1)
    base.update(kw)
    d = oracle.make_inputs(1, **base)
    x, B, dt, dA = (_dev(d[k]) for k in ("x", "B", "dt", "dA_cumsum"))
    b, L, H, P = x.shape
    C, N = dt.shape[2], B.shape[-1]
    out = torch.full((b, C, H, P, N), float("nan"), device="cuda")
    fin = torch.full((b, H, P, N), float("nan"), device="cuda")
    ops.measure_traffic_floor(B, x, dt, dA, out, fin)
    torch.cuda.synchronize()
    assert int((out != 0).sum()) == 0
    assert bool(torch.isnan(fin).all())
    # one side of the traffic alone: the loads leave `out` as it is, the stores write all of it
    out.fill_(float("nan"))
    ops.measure_traffic_floor(B, x, dt, dA, out, fin, part=1)
    torch.cuda.synchronize()
    assert bool(torch.isnan(out).all())
    ops.measure_traffic_floor(B, x, dt, dA, out, fin, part=2)
    torch.cuda.synchronize()
    assert int((out != 0).sum()) == 0
    with pytest.raises(RuntimeError):
        ops.measure_traffic_floor(B, x, dt, dA, out, fin, part=3)
    with pytest.raises(RuntimeError):                      # fp32 inputs are not the chain kernel's: no floor defined
        ops.measure_traffic_floor(B.float(), x.float(), dt, dA, out, fin)
