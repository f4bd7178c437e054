#!/usr/bin/env python3
"""SDDMM benchmark: GFLOP/s (2*nnz*K) and fraction of the HBM roofline, fp32.

One "step" is one sddmm_execute over the whole synthetic matrix with indices,
values, W and H resident in HBM and the output left on the device.  Default
workload: the recommender-ratings shape (480,189 x 17,770, ~100M nnz, K = 128).
Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps 1000] [--warmup 100] [--config 3] [--K 128]
                  [--kernel auto|row|lds|panel|hybrid] [--tile-x X] [--tile-y Y] [--spinup-ms 300]
                  [--no-sweep] [--no-cpu] [--copy-probe]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published

# HBM bytes per step measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on
# the default workload (see profiles/*hbm_traffic*.txt for the runs and the
# copy-kernel scale factors); None where no such measurement exists.
MEASURED_TRAFFIC = {(3, 1.0, 128, "auto", 0, 0): 3.14e9}


def alg_bytes(nnz, n_rows, K, rows_touched, cols_touched):
    """Compulsory bytes, CSR form: col index + S.val + out per nonzero, the row
    pointers, and every touched W row and H row once."""
    return 12.0 * nnz + 4.0 * (n_rows + 1) + 4.0 * K * (rows_touched + cols_touched)


def time_steps(run, steps, warmup, torch, spinup_ms=0.0):
    stream = torch.cuda.current_stream()
    # untimed: bring the device out of its idle clocks (the first few dozen milliseconds of
    # work after an idle period run slower), then the W warm-up steps proper
    t_end = time.perf_counter() + spinup_ms * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(10):
            run(stream.cuda_stream)
        torch.cuda.synchronize()
    for _ in range(warmup):
        run(stream.cuda_stream)
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for a, b in evs:
        a.record(stream)  # HIP events on the stream the kernels are launched on
        run(stream.cuda_stream)
        b.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per = sorted(a.elapsed_time(b) for a, b in evs)
    return wall_ms / steps, sum(per) / len(per), per[len(per) // 2]


def cpu_baseline(d, K, budget_s=12.0):
    """The CPU oracle's OpenMP COO loop (the reference's CPU path restated, with
    the S.val factor applied) on a bounded leading slice of the same workload,
    on all host threads the box grants."""
    from oracle import oracle
    threads = oracle.max_threads()
    W = d["W"].cpu().numpy()
    H = d["H"].cpu().numpy()
    nnz = d["nnz"]

    def run(n):
        r = d["row_ind"][:n].cpu().numpy(); c = d["col_ind"][:n].cpu().numpy(); v = d["val"][:n].cpu().numpy()
        best = None
        for _ in range(2):
            _, sec = oracle.sddmm_coo(r, c, v, W, H, nthreads=threads, apply_val=True, timed=True)
            best = sec if best is None else min(best, sec)
        return best

    n0 = min(nnz, 1_000_000)
    t = run(n0)
    rate = n0 / max(t, 1e-9)
    n = int(min(nnz, max(n0, rate * budget_s / 2)))
    if n > n0:
        t = run(n)
    gflops = 2.0 * n * K / t / 1e9
    return dict(value=round(gflops, 3), unit="GFLOP/s", cores=threads, kind="port",
                sample=f"first {n} of {nnz} nonzeros (rows in order), K={K}, best of 2 runs, {t * 1e3:.1f} ms")


KERNEL_NAMES = {1: "row_gather", 2: "lds_tile", 3: "panel", 4: "hybrid", 5: "dense_block"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a step takes about a millisecond: the defaults time one second of steady state
    # (the first few dozen steps after an idle period run at lower clocks)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--spinup-ms", type=float, default=300.0,
                    help="untimed executes before the warm-up steps, to leave the idle clocks (0 = none)")
    ap.add_argument("--config", type=int, default=3)
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--K", type=int, default=None)
    ap.add_argument("--kernel", default="auto", choices=["auto", "row", "lds", "panel", "hybrid"])
    ap.add_argument("--epilogue", default="scale", choices=["scale", "residual"],
                    help="scale: out = val*dot (the reference's form, the default); residual: out = val - dot, fused")
    ap.add_argument("--tile-x", type=int, default=0)
    ap.add_argument("--tile-y", type=int, default=0)
    ap.add_argument("--no-sweep", action="store_true", help="skip the K = 32, 128, 256, 512 report")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 1 GiB device copy (a known-size reference for HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)

    import torch
    from sddmm_gpu_amd import capi, synth
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    kernel = {"auto": capi.KERNEL_AUTO, "row": capi.KERNEL_ROW_GATHER, "lds": capi.KERNEL_LDS_TILE,
              "panel": capi.KERNEL_PANEL, "hybrid": capi.KERNEL_HYBRID}[args.kernel]
    names = {1: "uniform 4096^2 1%", 2: "bag-of-words 1500x12419", 3: "recommender 480189x17770 ~100M nnz",
             4: "R-MAT 2^22 ~200M nnz", 5: "banded 2^20 64/row"}

    d = synth.make(args.config, args.scale, device=dev, K=args.K)
    K0 = d["K"]
    sigma = float(d["W"].std())

    def set_rank(K):
        if K != d["K"]:
            g = torch.Generator(device=dev); g.manual_seed(1000 + K)
            d["W"] = torch.randn(d["n_rows"], K, generator=g, device=dev) * sigma
            d["H"] = torch.randn(d["n_cols"], K, generator=g, device=dev) * sigma
            d["K"] = K

    def measure(K):
        set_rank(K)
        plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], d["row_ptr"].data_ptr(),
                                         d["col_ind"].data_ptr(), K, args.tile_x, args.tile_y, kernel)
        info = plan.info()
        out = torch.empty(d["nnz"], device=dev)
        # S.val belongs to the matrix like its indices: it is handed to the plan once,
        # outside the timed region; W and H are the per-step inputs
        plan.set_values(d["val"].data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        vp, wp, hp, op = 0, d["W"].data_ptr(), d["H"].data_ptr(), out.data_ptr()
        epi = capi.EPILOGUE_RESIDUAL if args.epilogue == "residual" else capi.EPILOGUE_SCALE
        run = (lambda s: plan.execute(vp, wp, hp, op, s)) if args.epilogue == "scale" else \
              (lambda s: plan.execute_epilogue(vp, wp, hp, op, epi, s))
        wall, mean_ev, med_ev = time_steps(run, args.steps, args.warmup, torch,
                                           args.spinup_ms)
        prof = plan.execute_profiled(vp, wp, hp, op, torch.cuda.current_stream().cuda_stream)
        flops = 2.0 * d["nnz"] * K
        balg = alg_bytes(d["nnz"], d["n_rows"], K, info["rows_touched"], info["cols_touched"])
        res = dict(K=K, ms_per_step=wall, kernel_ms_mean=mean_ev, kernel_ms_median=med_ev,
                   gflops=flops / (wall * 1e6), alg_bytes=balg, alg_gbps=balg / (mean_ev * 1e6),
                   frac=balg / (mean_ev * 1e6) / HBM_PEAK_GBPS, info=info, prof=prof)
        plan.close()
        return res

    main_res = measure(K0)
    info = main_res["info"]
    line = {
        "metric": "SDDMM GFLOP/s (2*nnz*K), fp32",
        "value": round(main_res["gflops"], 2),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_res["ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": names[args.config] + (f" (scale {args.scale})" if args.scale != 1.0 else ""),
                   "n_rows": d["n_rows"], "n_cols": d["n_cols"], "nnz": d["nnz"], "K": K0, "seed": d["seed"],
                   "kernel": KERNEL_NAMES[info["kernel"]], "tile_size_x": info["tile_size_x"],
                   "tile_size_y": info["tile_size_y"], "k_slice": info["k_slice"],
                   "kernel_launches_per_step": info["n_launches"], "plan_ms": round(info["plan_ms"], 1),
                   "spinup_ms": args.spinup_ms, "epilogue": args.epilogue},
        "roofline": {"bound": "hbm", "achieved": round(main_res["alg_gbps"], 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(main_res["frac"], 4),
                     "traffic": MEASURED_TRAFFIC.get((args.config, args.scale, K0, args.kernel, args.tile_x, args.tile_y)),
                     "alg_bytes_per_step": main_res["alg_bytes"], "kernel_ms": round(main_res["kernel_ms_mean"], 5),
                     "kernels": [{"kernel": KERNEL_NAMES[p["kernel"]], "lanes_per_nnz": p["lanes_per_nnz"],
                                  "k_slice": p["k_slice"], "launches": p["n_kernel_launches"], "nnz": p["nnz"],
                                  "rows": p["rows"], "stream_positions": p["stream_positions"],
                                  "ms": round(p["ms"], 5)} for p in main_res["prof"]]},
    }
    if not args.no_sweep and args.config == 3:
        sweep = {}
        for K in (32, 128, 256, 512):
            r = main_res if K == K0 else measure(K)
            sweep[str(K)] = {"gflops": round(r["gflops"], 1), "kernel_ms": round(r["kernel_ms_mean"], 4),
                             "hbm_frac": round(r["frac"], 4)}
        line["gflops_by_K"] = sweep
    # a plain 1 GiB device-to-device copy next to it: with --copy-probe as the known-size
    # reference for the HBM counters, always as the bandwidth a streaming kernel reaches here
    n = 1 << 30
    a = torch.empty(n // 4, device=dev); b = torch.empty_like(a)
    a.fill_(1.0)
    b.copy_(a)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        b.copy_(a)
    e1.record()
    torch.cuda.synchronize()
    line["roofline"]["measured_copy_gbps"] = round(10 * 2.0 * n / (e0.elapsed_time(e1) * 1e6), 1)
    if args.copy_probe:
        line["copy_probe_bytes_each_way"] = n
    del a, b
    if not args.no_cpu:
        set_rank(K0)
        line["cpu_baseline"] = cpu_baseline(d, K0)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
