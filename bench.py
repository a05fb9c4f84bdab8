#!/usr/bin/env python3
"""Benchmark of the fused SSD chunk-state + state-passing path on one MI355X.

One "step" = one fused launch over one batch of synthetic input (default workload: the Mamba2-2.7B layer
shape, b=4, L=8192, H=80, P=64, N=128, chunk 256, bf16 inputs, fp32 states, fp32 initial states).
Prints ONE JSON line on stdout; details go to stderr.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 0..4] [--no-cpu]
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
# HBM bytes per fused launch measured with rocprofv3 --pmc (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, KiB -> bytes; the
# factors are what the same counters read for a plain 1 GiB copy).  Keyed by workload name; see the rocprof summaries
# kept with the repository.  None = not measured for that workload / kernel version.
MEASURED_TRAFFIC_BYTES = {"cfg2_mamba2_2p7b": 730515354}
MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--sets", type=int, default=3, help="rotating input/output buffer sets (defeats cache reuse)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline leg")
    ap.add_argument("--with-states", action="store_true", help="also materialise the per-chunk states")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 1 GiB device copy three times (the known-size kernel that the FETCH_SIZE / "
                         "WRITE_SIZE counters are scaled by) and exit")
    args = ap.parse_args()
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

    def timed(fn, steps, warmup):
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
    unf_wall, unf_ev = timed(unfused, max(5, args.steps // 4), 3)

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

    # the consumer of the passed states (state half of the chunk scan), fp32 y, on the states of the timed launches
    C_dev = [mv(d["C"]).clone() for _ in range(nsets)]
    prev_states = [fused(i)[0] for i in range(nsets)]
    y_bufs = [torch.empty(b, L, H, P, device=dev) for _ in range(nsets)]

    def scan_states(i):
        s = sets[i % nsets]
        return ssd_amd._chunk_scan_states_fwd(C_dev[i % nsets], prev_states[i % nsets], s["dA_cumsum"], seq_idx=s["seq_idx"],
                                              out=y_bufs[i % nsets])

    _, bf16_ev = timed(fused_bf16, max(5, args.steps // 4), 3)
    _, cs_ev = timed(cumsum, max(5, args.steps // 4), 3)
    _, scan_ev = timed(scan_states, max(5, args.steps // 4), 3)
    del prev_states, y_bufs

    # parity of what was timed, on one batch row, against the CPU oracle
    out, fin = fused(0)
    torch.cuda.synchronize()
    sl = slice(0, 1)
    cut = lambda t: None if t is None else t[sl]
    w_out, w_fin = ssd_oracle.fused_ref(d["B"][sl], d["x"][sl], d["dt"][sl], d["dA_cumsum"][sl],
                                        initial_states=cut(d["initial_states"]), seq_idx=cut(d["seq_idx"]))
    err = (out[sl].cpu() - w_out).abs()
    bad = int((err > 1e-3 + 2e-3 * w_out.abs()).sum()) + int(((fin[sl].cpu() - w_fin).abs() > 1e-3 + 2e-3 * w_fin.abs()).sum())
    log(f"[bench] parity (batch row 0): max|err|={float(err.max()):.3e}, mismatches={bad}")

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
                     "traffic": None if args.with_states else MEASURED_TRAFFIC_BYTES.get(cfg["name"]),
                     "algorithmic_bytes": alg_bytes, "kernel_us": round(ev_step * 1e6, 2)},
        "tflops": round(alg_flops / ev_step / 1e12, 2),
        "mfma_frac_of_bf16_peak": round(2 * alg_flops / ev_step / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
        "unfused_us": round(unf_ev * 1e6, 2),
        "fused_bf16_out_us": round(bf16_ev * 1e6, 2),
        "chunk_cumsum_us": round(cs_ev * 1e6, 2),
        "chunk_scan_states_us": round(scan_ev * 1e6, 2),
        "fused_speedup_vs_unfused": round(unf_ev / ev_step, 3),
        "parity_mismatches": bad,
    }

    if not args.no_cpu:
        # reference math in fp32 PyTorch on this machine's host cores: one batch row of the workload
        # (a bounded sample), scaled to the full layer
        nthreads = torch.get_num_threads()
        args_cpu = (d["B"][sl], d["x"][sl], d["dt"][sl], d["dA_cumsum"][sl])
        kw_cpu = dict(initial_states=cut(d["initial_states"]), seq_idx=cut(d["seq_idx"]))
        ssd_oracle.fused_ref(*args_cpu, **kw_cpu)
        ts = []
        for _ in range(2):
            t0 = time.perf_counter()
            ssd_oracle.fused_ref(*args_cpu, **kw_cpu)
            ts.append(time.perf_counter() - t0)
        cpu_s = sorted(ts)[0] * b
        res["cpu_baseline"] = {"value": round(cpu_s * 1e6, 1), "unit": "us/layer", "cores": nthreads, "kind": "port",
                               "sample": f"fp32 PyTorch restatement of the reference math (oracle/ssd_oracle.py fused_ref) on batch "
                                         f"row 0 of {b}, best of 2, scaled x{b}; torch threads={nthreads}, os.cpu_count()={os.cpu_count()}"}
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
