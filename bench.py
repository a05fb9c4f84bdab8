#!/usr/bin/env python3
"""Benchmark of the fused SSD chunk-state + state-passing path on one MI355X.

One "step" = one fused launch over one batch of synthetic input (default workload: the Mamba2-2.7B layer
shape, b=4, L=8192, H=80, P=64, N=128, chunk 256, bf16 inputs, fp32 states, fp32 initial states).
Prints ONE JSON line on stdout; details go to stderr.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--ramp-ms MS] [--config 0..4] [--no-cpu] [--no-per-config]

Every timed measurement is preceded by `--ramp-ms` (default 300) milliseconds of the same call, untimed, then the W
warm-up steps: after host-side work (input generation, parity checks) the GPU sits at low-power clocks and needs about
50 ms of load to leave them -- the first 100 launches of a cold series run 10 - 25 % slower than the 700 that follow.
The timed region is exactly K steps between two synchronisations.

Besides the headline workload the line carries `per_config`: the fused call timed the same way on each of the five
benchmark configurations (microseconds, GB/s of algorithmic bytes, fraction of HBM peak, TFLOP/s, parity mismatches
against the CPU oracle).  `roofline.plain_copy_gbps` is what a device-to-device copy of the same number of bytes (half
read, half written) reaches in the same run, timed the same way, and `roofline.frac_of_plain_copy` the fused call's
rate as a fraction of it: the published peak is not reachable by any kernel that reads and writes.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0           # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
# HBM bytes per fused launch measured with rocprofv3 --pmc (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, KiB -> bytes; the
# factors are what the same counters read for a plain 1 GiB copy), keyed by workload name, together with the hash of
# the kernel sources the measurement was made on (kernel_source_hash() below).  The counters cannot be read from
# inside this script, so the figure is only reported while the sources still hash to the same value; otherwise
# `roofline.traffic` is null.  The rocprof summaries are kept with the repository.
MEASURED_TRAFFIC = {
    "cfg1_mamba2_130m": {"bytes": 114583516, "sources": "c6fd050c8b07c621"},
    "cfg2_mamba2_2p7b": {"bytes": 812925361, "sources": "c6fd050c8b07c621"},
    "cfg3_varlen_packed": {"bytes": 831817499, "sources": "c6fd050c8b07c621"},
    "cfg4_long_grouped": {"bytes": 5367196082, "sources": "c6fd050c8b07c621"},
}
KERNEL_SOURCES = ("ssd_chain_kernel.h", "ssd_chain.hip", "ssd_quad.hip", "ssd_mfma.hip", "ssd_tile.h", "ssd_params.h", "ssd_capi.hip")


def kernel_source_hash():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "mamba-fused-minimal_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    m = MEASURED_TRAFFIC.get(workload)
    return m["bytes"] if m and m["sources"] == kernel_source_hash() else None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--ramp-ms", type=float, default=300.0,
                    help="before every timed measurement (and before its W warm-up steps) the measured call is repeated "
                         "for this long, untimed: the GPU leaves its low-power clocks only after about 50 ms of load "
                         "(0 = off)")
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--sets", type=int, default=3, help="rotating input/output buffer sets (defeats cache reuse)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline leg")
    ap.add_argument("--no-per-config", action="store_true", help="skip the table over the five configurations")
    ap.add_argument("--source-hash", action="store_true", help="print the hash of the kernel sources and exit")
    ap.add_argument("--with-states", action="store_true", help="also materialise the per-chunk states")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 1 GiB device copy three times (the known-size kernel that the FETCH_SIZE / "
                         "WRITE_SIZE counters are scaled by) and exit")
    args = ap.parse_args()
    if args.source_hash:
        print(kernel_source_hash())
        return
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU only (the driver's boxes have one GPU, and the path needs "
              "no exchange across GPUs); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from __graft_entry__ import ensure_built
    ensure_built()
    import ssd_amd
    from oracle import ssd_oracle          # input recipe + the cpu_baseline leg only

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    dev = torch.device("cuda:0")
    if args.copy_calibration:
        a = torch.ones(1 << 28, dtype=torch.float32, device=dev)      # 1 GiB
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": "3 x copy of 1073741824 bytes (1048576 KiB read, 1048576 KiB written each)"}))
        return
    cfg = ssd_oracle.CONFIGS[args.config]
    log(f"[bench] workload {cfg['name']}: {cfg}")
    d = ssd_oracle.make_inputs(args.config)
    mv = lambda t: None if t is None else t.to(dev)
    base = {k: mv(d[k]) for k in ("B", "x", "dt", "dA_cumsum", "initial_states", "seq_idx")}
    nsets = max(1, args.sets)
    sets = [base] + [{k: (None if v is None else v.clone()) for k, v in base.items()} for _ in range(nsets - 1)]
    b, L, H, P = d["x"].shape
    N, C = d["B"].shape[-1], d["dt"].shape[2]
    st_bufs = [torch.empty(b, C, H, P, N, device=dev) if args.with_states else None for _ in range(nsets)]

    def fused(i):
        s = sets[i % nsets]
        return ssd_amd._fused_chunk_state_state_passing_fwd(
            s["B"], s["x"], s["dt"], s["dA_cumsum"], torch.float32, initial_states=s["initial_states"],
            seq_idx=s["seq_idx"], states=st_bufs[i % nsets])

    def unfused(i):
        s = sets[i % nsets]
        st = ssd_amd._chunk_state_fwd(s["B"], s["x"], s["dt"], s["dA_cumsum"], seq_idx=s["seq_idx"])
        init = None if s["initial_states"] is None else s["initial_states"].flatten(-2)
        return ssd_amd._state_passing_fwd(st.flatten(-2), s["dA_cumsum"][:, :, :, -1], initial_states=init,
                                          seq_idx=s["seq_idx"], chunk_size=cfg["Q"])

    def ramp(fn):
        t0, i = time.perf_counter(), 0
        while (time.perf_counter() - t0) * 1e3 < args.ramp_ms:
            for _ in range(20):
                fn(i)
                i += 1
            torch.cuda.synchronize()

    def timed(fn, steps, warmup):
        ramp(fn)
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(steps):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        return wall / steps, e0.elapsed_time(e1) * 1e-3 / steps     # seconds per step (host clock, device events)

    wall_step, ev_step = timed(fused, args.steps, args.warmup)
    # a failed chain (a wait that ran out, an XCD without a workgroup ...) leaves outputs unusable and says so only here
    chain_status = ssd_amd.fused_status()
    assert chain_status == 0, f"the fused launches report status {chain_status}"
    # every figure beside the headline is an average over at least 20 launches, whatever --steps is
    steps_2nd = max(20, args.steps // 4)
    unf_wall, unf_ev = timed(unfused, steps_2nd, 3)

    # neighbours of the path, reported beside the headline: the fused call with bf16 passed states (what the
    # reference's main.py asks for, out_dtype = C.dtype) and the producer of dt / dA_cumsum
    def fused_bf16(i):
        s = sets[i % nsets]
        return ssd_amd._fused_chunk_state_state_passing_fwd(
            s["B"], s["x"], s["dt"], s["dA_cumsum"], torch.bfloat16, initial_states=s["initial_states"],
            seq_idx=s["seq_idx"])

    raw = [mv(d["dt_raw"]).clone() for _ in range(nsets)]
    A_dev, bias_dev = mv(d["A"]), mv(d["dt_bias"])

    def cumsum(i):
        return ssd_amd._chunk_cumsum_fwd(raw[i % nsets], A_dev, cfg["Q"], dt_bias=bias_dev, dt_softplus=True)

    # producer + path in one call (two launches: the producer's clears the chain kernel's workspace on its way)
    def prep_fused(i):
        s = sets[i % nsets]
        return ssd_amd._fused_cumsum_chunk_state_state_passing_fwd(
            s["B"], s["x"], raw[i % nsets], A_dev, cfg["Q"], torch.float32, dt_bias=bias_dev, dt_softplus=True,
            initial_states=s["initial_states"], seq_idx=s["seq_idx"])

    # the consumer of the passed states (state half of the chunk scan), fp32 y, on the states of the timed launches
    C_dev = [mv(d["C"]).clone() for _ in range(nsets)]
    prev_states = [fused(i)[0] for i in range(nsets)]
    y_bufs = [torch.empty(b, L, H, P, device=dev) for _ in range(nsets)]

    def scan_states(i):
        s = sets[i % nsets]
        return ssd_amd._chunk_scan_states_fwd(C_dev[i % nsets], prev_states[i % nsets], s["dA_cumsum"], seq_idx=s["seq_idx"],
                                              out=y_bufs[i % nsets])

    # what the part's memory system gives a kernel with nothing else to do: a device-to-device copy that reads half of
    # the path's algorithmic bytes and writes the other half (the path reads x and writes `out`, about as much)
    half = ssd_oracle.algorithmic_bytes(cfg, with_states=args.with_states) // 2
    cp_src = [torch.empty(half, dtype=torch.uint8, device=dev).random_() for _ in range(nsets)]
    cp_dst = [torch.empty(half, dtype=torch.uint8, device=dev) for _ in range(nsets)]

    def plain_copy(i):
        cp_dst[i % nsets].copy_(cp_src[i % nsets])

    _, copy_ev = timed(plain_copy, steps_2nd, 3)
    del cp_src, cp_dst

    # ... and a kernel with this path's own streams and nothing else: x and B rows in, one fp32 state tile per (state
    # tile, chunk) out, no arithmetic, no chain (ssd_measure_traffic_floor; it overwrites the `out` it is given)
    mover_ev = mover_ld_ev = mover_st_ev = None
    if cfg["dtype"] == "bf16" and not args.with_states:
        mv_out = [torch.empty(b, C, H, P, N, device=dev) for _ in range(nsets)]
        mv_fin = torch.empty(b, H, P, N, device=dev)

        def mover(i, part=0):
            s = sets[i % nsets]
            ssd_amd.measure_traffic_floor(s["B"], s["x"], s["dt"], s["dA_cumsum"], mv_out[i % nsets], mv_fin, part)

        try:
            _, mover_ev = timed(mover, steps_2nd, 3)
            # ... and each side of its traffic alone: how reads and writes share the memory system
            _, mover_ld_ev = timed(lambda i: mover(i, 1), steps_2nd, 3)
            _, mover_st_ev = timed(lambda i: mover(i, 2), steps_2nd, 3)
        except RuntimeError as e:          # a shape the chain kernel does not cover has no such floor
            log(f"[bench] no traffic floor for this workload: {e}")
        del mv_out, mv_fin
    _, bf16_ev = timed(fused_bf16, steps_2nd, 3)
    _, cs_ev = timed(cumsum, steps_2nd, 3)
    _, prep_ev = timed(prep_fused, steps_2nd, 3)
    _, scan_ev = timed(scan_states, steps_2nd, 3)
    # ... and on bf16 passed states (the reference's main.py hands its scan `out` in C's type)
    prev_states = [fused_bf16(i)[0] for i in range(nsets)]
    _, scan16_ev = timed(scan_states, steps_2nd, 3)
    del prev_states
    # path + consumer in one launch (ssd_fused_chunk_state_passing_scan_fwd): with the passed states as an output and
    # fp32 y -- what the two calls above compute together --, and without them (bf16 y, the type the reference's scan
    # writes; fp32 y), where they never reach memory
    fscan = {}
    if cfg["dtype"] == "bf16" and not args.with_states:
        y16 = [torch.empty(b, L, H, P, device=dev, dtype=torch.bfloat16) for _ in range(nsets)]

        def make(ret, ybufs, kern=0):
            def f(i):
                s = sets[i % nsets]
                return ssd_amd._fused_chunk_state_state_passing_scan_fwd(
                    s["B"], s["x"], C_dev[i % nsets], s["dt"], s["dA_cumsum"], torch.float32, initial_states=s["initial_states"],
                    seq_idx=s["seq_idx"], y=ybufs[i % nsets], return_states=ret, _kernel=kern)
            return f

        # headline of the one-launch entry: no passed states in memory, y in the type the reference's scan writes
        # (C's: bf16); then fp32 y; then with `out` as well, which the library runs as its two stand-alone calls
        # unless the one-launch kernel is insisted on (last figure)
        for key, ret, ybufs, kern in (("fused_with_scan_states_us", False, y16, 0), ("fused_with_scan_states_fp32_y_us", False, y_bufs, 0),
                                      ("fused_with_scan_states_and_out_fp32_y_us", True, y_bufs, 0),
                                      ("fused_with_scan_states_and_out_one_launch_us", True, y_bufs, 1)):
            _, ev = timed(make(ret, ybufs, kern), steps_2nd, 3)
            assert ssd_amd.fused_status() == 0
            fscan[key] = round(ev * 1e6, 2)
        # parity of the last variant against the oracle on one batch row
        o_, f_, y_ = make(False, y16)(0)
        torch.cuda.synchronize()
        wo, wf = ssd_oracle.fused_ref(d["B"][:1], d["x"][:1], d["dt"][:1], d["dA_cumsum"][:1],
                                      initial_states=None if d["initial_states"] is None else d["initial_states"][:1],
                                      seq_idx=None if d["seq_idx"] is None else d["seq_idx"][:1])
        wy = ssd_oracle.chunk_scan_states_ref(d["C"][:1], wo, d["dA_cumsum"][:1], seq_idx=None if d["seq_idx"] is None else d["seq_idx"][:1])
        ey = (y_[:1].float().cpu() - wy).abs()
        fscan["fused_scan_parity_mismatches"] = int((ey > 1e-3 + (2e-3 + 2.0 ** -8) * wy.abs()).sum())
        del y16, o_, f_, y_
    del y_bufs
    # the headline call again without the clock ramp, right after host-side idling: what a lone call in a quiet stream sees
    torch.cuda.synchronize()
    time.sleep(0.5)
    saved_ramp, args.ramp_ms = args.ramp_ms, 0.0
    _, cold_ev = timed(fused, 20, 0)
    args.ramp_ms = saved_ramp

    # parity of what was timed, over the whole batch, against the CPU oracle (the long grouped configuration on four
    # heads of different groups: its fp32 oracle would not fit a few minutes)
    def parity(idx, dd, out, fin):
        if idx == 4:
            ratio, bad, worst = dd["x"].shape[2] // dd["B"].shape[2], 0, 0.0
            for h in (0, 17, 63, 127):
                g = h // ratio
                wo, wf = ssd_oracle.fused_ref(dd["B"][:, :, g:g + 1], dd["x"][:, :, h:h + 1], dd["dt"][:, h:h + 1], dd["dA_cumsum"][:, h:h + 1])
                eo, ef = (out[:, :, h:h + 1].cpu() - wo).abs(), (fin[:, h:h + 1].cpu() - wf).abs()
                bad += int((eo > 1e-3 + 2e-3 * wo.abs()).sum()) + int((ef > 1e-3 + 2e-3 * wf.abs()).sum())
                worst = max(worst, float(eo.max()), float(ef.max()))
            return bad, worst, "heads 0, 17, 63, 127"
        wo, wf = ssd_oracle.fused_ref(dd["B"], dd["x"], dd["dt"], dd["dA_cumsum"], initial_states=dd["initial_states"], seq_idx=dd["seq_idx"])
        eo, ef = (out.cpu() - wo).abs(), (fin.cpu() - wf).abs()
        bad = int((eo > 1e-3 + 2e-3 * wo.abs()).sum()) + int((ef > 1e-3 + 2e-3 * wf.abs()).sum())
        return bad, max(float(eo.max()), float(ef.max())), "whole batch"

    out, fin = fused(0)
    torch.cuda.synchronize()
    bad, worst, scope = parity(args.config, d, out, fin)
    log(f"[bench] parity ({scope}): max|err|={worst:.3e}, mismatches={bad}")
    del out, fin

    alg_bytes = ssd_oracle.algorithmic_bytes(cfg, with_states=args.with_states)
    alg_flops = ssd_oracle.algorithmic_flops(cfg)
    achieved = alg_bytes / ev_step / 1e9
    res = {
        "metric": "fused chunk-state+state-passing us/layer",
        "value": round(wall_step * 1e6, 2),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "clock_ramp_ms": args.ramp_ms,
        "ms_per_step": round(wall_step * 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if cfg["dtype"] == "bf16" else cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": f"{cfg['name']}: b={b} L={L} nheads={H} headdim={P} dstate={N} ngroups={cfg['G']} chunk={cfg['Q']}"
                               f"{' +initial_states' if cfg['init'] else ''}{' varlen seq_idx' if cfg['nseq'] else ''}, "
                               f"{cfg['dtype']} x/B, fp32 dt/dA_cumsum/out/final",
                   "materialise_states": bool(args.with_states), "buffer_sets": nsets},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": None if args.with_states else measured_traffic(cfg["name"]),
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on the kernel sources with hash "
                                       + kernel_source_hash() + " (null: not measured on these sources)",
                     "algorithmic_bytes": alg_bytes, "kernel_us": round(ev_step * 1e6, 2),
                     "plain_copy_us": round(copy_ev * 1e6, 2), "plain_copy_gbps": round(2 * half / copy_ev / 1e9, 1),
                     "frac_of_plain_copy": round(copy_ev * 2 * half / alg_bytes / ev_step, 4),
                     "mover_us": None if mover_ev is None else round(mover_ev * 1e6, 2),
                     "mover_bytes": None if mover_ev is None else b * L * H * P * 2 + d["B"].numel() * 2 + b * C * H * P * N * 4,
                     "frac_of_mover": None if mover_ev is None else round(mover_ev / ev_step, 4),
                     "mover_loads_us": None if mover_ld_ev is None else round(mover_ld_ev * 1e6, 2),
                     "mover_stores_us": None if mover_st_ev is None else round(mover_st_ev * 1e6, 2),
                     "kernel_us_cold": round(cold_ev * 1e6, 2), "frac_cold": round(alg_bytes / cold_ev / 1e9 / HBM_PEAK_GBPS, 4)},
        "tflops": round(alg_flops / ev_step / 1e12, 2),
        "mfma_frac_of_bf16_peak": round(2 * alg_flops / ev_step / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
        "unfused_us": round(unf_ev * 1e6, 2),
        "fused_bf16_out_us": round(bf16_ev * 1e6, 2),
        "chunk_cumsum_us": round(cs_ev * 1e6, 2),
        "fused_with_dt_preparation_us": round(prep_ev * 1e6, 2),
        "chunk_scan_states_us": round(scan_ev * 1e6, 2),
        "chunk_scan_states_from_bf16_us": round(scan16_ev * 1e6, 2),
        **fscan,
        "fused_speedup_vs_unfused": round(unf_ev / ev_step, 3),
        "parity_mismatches": bad,
        "parity_scope": scope,
    }

    if not args.no_per_config:
        # the same call, timed the same way, on each of the five configurations
        table = {}
        steps_pc = steps_2nd
        for idx in range(5):
            c = ssd_oracle.CONFIGS[idx]
            if idx == args.config:
                dd, ev = d, ev_step
                o, f = fused(0)
                torch.cuda.synchronize()
                pbad, pworst, pscope = bad, worst, scope
            else:
                dd = ssd_oracle.make_inputs(idx)
                n = 2 if idx == 4 else nsets
                dev_sets = [{k: mv(dd[k]) for k in ("B", "x", "dt", "dA_cumsum", "initial_states", "seq_idx")}]
                dev_sets += [{k: (None if v is None else v.clone()) for k, v in dev_sets[0].items()} for _ in range(n - 1)]

                def call(i, dev_sets=dev_sets, n=n):
                    s_ = dev_sets[i % n]
                    return ssd_amd._fused_chunk_state_state_passing_fwd(
                        s_["B"], s_["x"], s_["dt"], s_["dA_cumsum"], torch.float32, initial_states=s_["initial_states"],
                        seq_idx=s_["seq_idx"])

                _, ev = timed(call, steps_pc, 3)
                o, f = call(0)
                torch.cuda.synchronize()
                pbad, pworst, pscope = parity(idx, dd, o, f)
                del dev_sets
            ab, af = ssd_oracle.algorithmic_bytes(c), ssd_oracle.algorithmic_flops(c)
            table[f"cfg{idx}"] = {"workload": c["name"], "us": round(ev * 1e6, 2), "gbps": round(ab / ev / 1e9, 1),
                                  "frac": round(ab / ev / 1e9 / HBM_PEAK_GBPS, 4), "tflops": round(af / ev / 1e12, 2),
                                  "algorithmic_bytes": ab, "parity_mismatches": pbad, "parity_scope": pscope}
            log(f"[bench] {c['name']}: {table[f'cfg{idx}']}")
            del o, f, dd
            torch.cuda.empty_cache()
        res["per_config"] = table

    if not args.no_cpu:
        # reference math in fp32 PyTorch on this machine's host cores: the whole batch of the workload, one warm-up
        # and three timed repetitions (the long grouped configuration: one repetition on 8 of its 128 heads, scaled)
        nthreads = torch.get_num_threads()
        if args.config == 4:
            hs, scale, reps = slice(0, 8), H / 8, 1
            args_cpu = (d["B"][:, :, 0:1], d["x"][:, :, hs], d["dt"][:, hs], d["dA_cumsum"][:, hs])
            what = f"heads 0-7 of {H}, 1 repetition, scaled x{H // 8}"
        else:
            scale, reps = 1.0, 3
            args_cpu = (d["B"], d["x"], d["dt"], d["dA_cumsum"])
            what = "the whole batch, 1 warm-up + 3 repetitions, median"
        kw_cpu = dict(initial_states=d["initial_states"] if args.config != 4 else None, seq_idx=d["seq_idx"])
        if reps > 1:
            ssd_oracle.fused_ref(*args_cpu, **kw_cpu)
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            ssd_oracle.fused_ref(*args_cpu, **kw_cpu)
            ts.append(time.perf_counter() - t0)
        cpu_s = sorted(ts)[len(ts) // 2] * scale
        res["cpu_baseline"] = {"value": round(cpu_s * 1e6, 1), "unit": "us/layer", "cores": nthreads, "kind": "port",
                               "sample": f"fp32 PyTorch restatement of the reference math (oracle/ssd_oracle.py fused_ref) on {what}; "
                                         f"torch threads={nthreads}, os.cpu_count()={os.cpu_count()}"}
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
