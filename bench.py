#!/usr/bin/env python3
"""SDDMM benchmark: GFLOP/s (2*nnz*K) and fraction of the HBM roofline, fp32.

One "step" is one sddmm_execute over the whole synthetic matrix with indices,
values, W and H resident in HBM and the output left on the device.  Default
workload: the recommender-ratings shape (480,189 x 17,770, ~100M nnz, K = 128).
Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps 1000] [--warmup 100] [--config 3] [--K 128]
                  [--kernel auto|row|lds|panel|hybrid] [--tile-x X] [--tile-y Y] [--spinup-ms 300]
                  [--opt field=value ...] [--no-sweep] [--no-cpu] [--no-parity] [--copy-probe]
                  [--tile-sweep] [--from-prof DIR]

--tile-sweep adds one row per tile configuration (tile_size_x x K slice x lanes per nonzero,
explicit values honoured) with its time, GB/s and launch shape; run under
rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE the same rows get their LDS
conflict counters (sddmm_gpu_amd/rocprof.py matches them by kernel variant, LDS size and grid).
--from-prof DIR merges such a profile (HBM bytes per step scaled by the copy probe, LDS bank
conflicts per active cycle, per-kernel durations) into the line; without it roofline.traffic is
read from the summary of the same workload kept under profiles/, whose name the line gives.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published



def traffic_profile_path(config, scale, K, kernel, tile_x, tile_y, opts):
    """Where the rocprofv3 summary with this workload's HBM bytes per step is kept (made by
    python -m sddmm_gpu_amd.rocprof from FETCH_SIZE / WRITE_SIZE passes of this script)."""
    if scale != 1.0 or tile_x or tile_y or opts:
        return None
    return os.path.join(ROOT, "profiles", f"hbm_traffic_config{config}_k{K}_{kernel}.txt")


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

    def run(n, reps):
        r = d["row_ind"][:n].cpu().numpy(); c = d["col_ind"][:n].cpu().numpy(); v = d["val"][:n].cpu().numpy()
        oracle.sddmm_coo(r, c, v, W, H, nthreads=threads, apply_val=True, timed=True)  # warm-up, not timed
        best = None
        for _ in range(reps):
            _, sec = oracle.sddmm_coo(r, c, v, W, H, nthreads=threads, apply_val=True, timed=True)
            best = sec if best is None else min(best, sec)
        return best

    n0 = min(nnz, 1_000_000)
    t = run(n0, 1)
    rate = n0 / max(t, 1e-9)
    n = int(min(nnz, max(n0, rate * budget_s / 4)))  # one warm-up + three timed runs inside the budget
    t = run(n, 3)
    gflops = 2.0 * n * K / t / 1e9
    model = "unknown CPU"
    try:
        for ln in open("/proc/cpuinfo"):
            if ln.startswith("model name"):
                model = ln.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return dict(value=round(gflops, 3), unit="GFLOP/s", cores=threads, kind="port",
                sample=f"first {n} of {nnz} nonzeros (rows in order), K={K}, one warm-up then best of 3 runs, "
                       f"{t * 1e3:.1f} ms, {threads} threads on {model}")


def parity_block(d, K, out, torch, n_sample=200_000):
    """A seeded sample of the nonzeros against the CPU oracle, outside the timed region: the
    strict count (|gpu - cpu| > 1e-5*sqrt(K)*|cpu|), the worst relative and norm-wise errors,
    the count under the bound the parity tests assert (relative, or norm-wise for nonzeros
    whose terms cancel), and how many of the oracle's own results miss the strict bound against
    an fp64 sum (what fp32 summation order alone costs on this input)."""
    import numpy as np
    from oracle import oracle
    g = torch.Generator(device=out.device); g.manual_seed(4242)
    n = min(n_sample, d["nnz"])
    idx = torch.randint(0, d["nnz"], (n,), generator=g, device=out.device)
    rows = d["row_ind"][idx].cpu().numpy(); cols = d["col_ind"][idx].cpu().numpy(); vals = d["val"][idx].cpu().numpy()
    # only the sampled rows of W and H travel to the host
    ur, ri = np.unique(rows, return_inverse=True); uc, ci = np.unique(cols, return_inverse=True)
    W = d["W"][torch.from_numpy(ur).to(out.device).long()].cpu().numpy()
    H = d["H"][torch.from_numpy(uc).to(out.device).long()].cpu().numpy()
    ri = ri.astype(np.int32); ci = ci.astype(np.int32)
    cpu = oracle.sddmm_coo(ri, ci, vals, W, H).astype(np.float64)
    f64, absp = oracle.sddmm_f64(ri, ci, vals, W, H)
    gpu = out[idx].cpu().numpy().astype(np.float64)
    tol = 1e-5 * np.sqrt(K)
    diff = np.abs(gpu - cpu)
    nz = np.abs(cpu) > 0; pos = absp > 0
    return dict(n_sample=int(n), tol=tol,
                strict_violations=int((diff > tol * np.abs(cpu)).sum()),
                max_rel=float((diff[nz] / np.abs(cpu[nz])).max()) if nz.any() else 0.0,
                max_normwise=float((diff[pos] / absp[pos]).max()) if pos.any() else 0.0,
                violations=int((diff > tol * np.maximum(np.abs(cpu), absp / 100.0)).sum()),
                cpu_vs_f64_strict=int((np.abs(cpu - f64) > tol * np.abs(f64)).sum()),
                gpu_vs_f64_strict=int((np.abs(gpu - f64) > tol * np.abs(f64)).sum()))


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
    ap.add_argument("--no-others", action="store_true", help="skip the other benchmark shapes (other_configs)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-parity", action="store_true", help="skip the sampled comparison with the CPU oracle")
    ap.add_argument("--opt", action="append", default=[], metavar="FIELD=VALUE",
                    help="a field of sddmm_plan_options (include/sddmm.h), e.g. --opt k_slice=64 --opt dense_blocks=1")
    ap.add_argument("--plan-file", default=None, metavar="PATH",
                    help="load the plan from PATH.k<K> when that file fits this matrix, K and options; otherwise build it and save it there")
    ap.add_argument("--tile-sweep", action="store_true", help="one row per tile configuration (see the module docstring)")
    ap.add_argument("--from-prof", default=None, metavar="DIR", help="merge a rocprofv3 profile of this workload into the line")
    ap.add_argument("--fused", action="store_true",
                    help="also time the forms around the SDDMM on the same workload: row softmax of out, SDDMM + softmax, SpMM")
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

    opt_fields = {}
    for kv in args.opt:
        k, _, v = kv.partition("=")
        opt_fields[k] = int(v)
    executes = [0]

    d = synth.make(args.config, args.scale, device=dev, K=args.K)
    K0 = d["K"]

    def set_rank(K, d=d):
        if K != d["K"]:
            g = torch.Generator(device=dev); g.manual_seed(1000 + K)
            s = float(d["W"].std())
            d["W"] = d["H"] = None
            d["W"] = torch.randn(d["n_rows"], K, generator=g, device=dev) * s
            d["H"] = torch.randn(d["n_cols"], K, generator=g, device=dev) * s
            d["K"] = K

    def measure(K, steps=None, warmup=None, spinup=None, keep_out=False, d=d, **more):
        set_rank(K, d)
        steps = args.steps if steps is None else steps
        warmup = args.warmup if warmup is None else warmup
        spinup = args.spinup_ms if spinup is None else spinup
        fields = dict(kernel=kernel, tile_size_x=args.tile_x, tile_size_y=args.tile_y)
        fields.update(opt_fields); fields.update(more)
        popt = capi.PlanOptions.defaults(**fields)
        plan, loaded = None, False
        if args.plan_file and not more:
            try:
                plan = capi.Plan.load_device(f"{args.plan_file}.k{K}", d["n_rows"], d["n_cols"], d["nnz"], d["row_ptr"].data_ptr(),
                                             d["col_ind"].data_ptr(), K, options=popt)
                loaded = True
            except capi.SddmmError as e:
                print(f"bench.py: no usable plan file ({e}); building the plan", file=sys.stderr)
        if plan is None:
            plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], d["row_ptr"].data_ptr(),
                                             d["col_ind"].data_ptr(), K, options=popt)
        info = plan.info()
        info["plan_loaded"] = loaded
        out = torch.empty(d["nnz"], device=dev)
        # S.val belongs to the matrix like its indices: it is handed to the plan once,
        # outside the timed region; W and H are the per-step inputs
        plan.set_values(d["val"].data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        if args.plan_file and not more and not loaded:
            plan.save(f"{args.plan_file}.k{K}")
        vp, wp, hp, op = 0, d["W"].data_ptr(), d["H"].data_ptr(), out.data_ptr()
        epi = capi.EPILOGUE_RESIDUAL if args.epilogue == "residual" else capi.EPILOGUE_SCALE

        def run(s):
            executes[0] += 1
            if args.epilogue == "scale":
                plan.execute(vp, wp, hp, op, s)
            else:
                plan.execute_epilogue(vp, wp, hp, op, epi, s)

        wall, mean_ev, med_ev = time_steps(run, steps, warmup, torch, spinup)
        prof = plan.execute_profiled(vp, wp, hp, op, torch.cuda.current_stream().cuda_stream)
        executes[0] += 1
        flops = 2.0 * d["nnz"] * K
        balg = alg_bytes(d["nnz"], d["n_rows"], K, info["rows_touched"], info["cols_touched"])
        res = dict(K=K, ms_per_step=wall, kernel_ms_mean=mean_ev, kernel_ms_median=med_ev,
                   gflops=flops / (wall * 1e6), alg_bytes=balg, alg_gbps=balg / (mean_ev * 1e6),
                   frac=balg / (mean_ev * 1e6) / HBM_PEAK_GBPS, info=info, prof=prof, options=plan.options())
        if wall < 0.1:
            # A launch-bound step: the same executes recorded once into a HIP graph (sddmm_execute only launches
            # kernels) and replayed, which is what a caller with such a loop would do.
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            n_rec = max(steps, 20)
            with torch.cuda.graph(g, stream=side):
                for _ in range(n_rec):
                    run(torch.cuda.current_stream().cuda_stream)
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(5):
                g.replay()
            torch.cuda.synchronize()
            res["graph_ms_per_step"] = (time.perf_counter() - t0) * 1e3 / (5 * n_rec)
            del g
        if keep_out:
            if args.epilogue != "scale":
                plan.execute(vp, wp, hp, op, torch.cuda.current_stream().cuda_stream)
                executes[0] += 1
            torch.cuda.synchronize()
            res["out"] = out
        plan.close()
        return res

    main_res = measure(K0, keep_out=not args.no_parity)
    info = main_res["info"]
    parity = None
    if not args.no_parity:
        parity = parity_block(d, K0, main_res.pop("out"), torch)
    tpath = traffic_profile_path(args.config, args.scale, K0, args.kernel, args.tile_x, args.tile_y, opt_fields)
    traffic = None
    if tpath:
        from sddmm_gpu_amd import rocprof
        traffic = rocprof.traffic_from_profile_text(tpath)
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
                   "kernel_launches_per_step": info["n_launches"], "plan_ms": round(info["plan_ms"], 1), "plan_loaded": info["plan_loaded"],
                   "graph_ms_per_step": round(main_res["graph_ms_per_step"], 5) if "graph_ms_per_step" in main_res else None,
                   "spinup_ms": args.spinup_ms, "epilogue": args.epilogue,
                   "dense_nnz": info["dense_nnz"], "dense_blocks": info["dense_blocks"],
                   "plan_options": {k: v for k, v in main_res["options"].items() if v not in (-1, 0) or k == "kernel"}},
        "roofline": {"bound": "hbm", "achieved": round(main_res["alg_gbps"], 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(main_res["frac"], 4),
                     "traffic": traffic,
                     "traffic_source": (os.path.relpath(tpath, ROOT) if traffic is not None else None),
                     "alg_bytes_per_step": main_res["alg_bytes"], "kernel_ms": round(main_res["kernel_ms_mean"], 5),
                     "kernels": [{"kernel": KERNEL_NAMES[p["kernel"]], "lanes_per_nnz": p["lanes_per_nnz"],
                                  "k_slice": p["k_slice"], "launches": p["n_kernel_launches"], "nnz": p["nnz"],
                                  "rows": p["rows"], "stream_positions": p["stream_positions"],
                                  "ms": round(p["ms"], 5)} for p in main_res["prof"]]},
    }
    if parity is not None:
        line["parity"] = parity
    if args.fused:
        # the callers' forms around the SDDMM, on the same matrix and rank: each timed like a step (HIP events on the
        # launch stream); algorithmic bytes: softmax reads and writes every entry once (8 nnz + the row pointers);
        # SpMM reads the pattern and its weights (8 nnz), the row pointers and the touched H rows and writes Y
        set_rank(K0)
        n_steps, n_warm = max(10, args.steps // 10), max(3, args.warmup // 10)
        x = torch.empty(d["nnz"], device=dev); y = torch.empty(d["nnz"], device=dev)
        plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], d["row_ptr"].data_ptr(), d["col_ind"].data_ptr(), K0,
                                         options=capi.PlanOptions.defaults(kernel=kernel, **opt_fields))
        plan.set_values(d["val"].data_ptr(), torch.cuda.current_stream().cuda_stream)
        plan.execute(0, d["W"].data_ptr(), d["H"].data_ptr(), x.data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        rp, ci = d["row_ptr"].data_ptr(), d["col_ind"].data_ptr()
        _, sm_ms, _ = time_steps(lambda st: capi.row_softmax(d["n_rows"], rp, x.data_ptr(), y.data_ptr(), st), n_steps, n_warm, torch, 30.0)
        _, es_ms, _ = time_steps(lambda st: plan.execute_softmax(0, d["W"].data_ptr(), d["H"].data_ptr(), y.data_ptr(), st),
                                 n_steps, n_warm, torch, 30.0)
        # the softmax of the full-size result against the same thing written with torch's segment operations
        torch.cuda.synchronize()
        ri = d["row_ind"].to(torch.int64)
        mx = torch.full((d["n_rows"],), float("-inf"), device=dev).scatter_reduce_(0, ri, x, "amax")
        ref = torch.exp(x - mx[ri])
        ref /= torch.zeros(d["n_rows"], device=dev).index_add_(0, ri, ref)[ri]
        sm_diff = float(((y - ref).abs() / ref.clamp_min(1e-37)).max())
        row_sums = torch.zeros(d["n_rows"], device=dev, dtype=torch.float64).index_add_(0, ri, y.double())
        sm_sum_dev = float((row_sums[row_sums > 0] - 1.0).abs().max())
        del ri, mx, ref, row_sums
        Y = torch.empty(d["n_rows"], K0, device=dev)
        _, sp_ms, _ = time_steps(lambda st: capi.spmm_csr(d["n_rows"], d["n_cols"], d["nnz"], rp, ci, y.data_ptr(), K0,
                                                          d["H"].data_ptr(), Y.data_ptr(), st), n_steps, n_warm, torch, 30.0)
        plan.close()
        # the same product on the plan's column tiles (spmm_stream = 1)
        plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], d["row_ptr"].data_ptr(), d["col_ind"].data_ptr(), K0,
                                         options=capi.PlanOptions.defaults(kernel=kernel, spmm_stream=1, **opt_fields))
        sp_info = plan.info()
        Y2 = torch.empty(d["n_rows"], K0, device=dev)
        _, spp_ms, _ = time_steps(lambda st: plan.spmm(y.data_ptr(), d["H"].data_ptr(), Y2.data_ptr(), 0, 0, st), n_steps, n_warm, torch, 30.0)
        torch.cuda.synchronize()
        sp_diff = float((Y2 - Y).abs().max() / Y.abs().max().clamp_min(1e-30))
        plan.close()
        del Y2
        sm_bytes = 8.0 * d["nnz"] + 4.0 * (d["n_rows"] + 1)
        sp_bytes = 8.0 * d["nnz"] + 4.0 * (d["n_rows"] + 1) + 4.0 * K0 * (info["cols_touched"] + d["n_rows"])
        line["fused"] = {
            "row_softmax": {"ms": round(sm_ms, 4), "alg_bytes": sm_bytes, "alg_gbps": round(sm_bytes / (sm_ms * 1e6), 1),
                            "hbm_frac": round(sm_bytes / (sm_ms * 1e6) / HBM_PEAK_GBPS, 4),
                            "max_rel_diff_vs_torch": sm_diff, "max_row_sum_minus_one": sm_sum_dev},
            "sddmm_plus_softmax": {"ms": round(es_ms, 4)},
            "spmm_csr": {"ms": round(sp_ms, 4), "gflops": round(2.0 * d["nnz"] * K0 / (sp_ms * 1e6), 1), "alg_bytes": sp_bytes,
                         "alg_gbps": round(sp_bytes / (sp_ms * 1e6), 1), "hbm_frac": round(sp_bytes / (sp_ms * 1e6) / HBM_PEAK_GBPS, 4)},
            "spmm_plan": {"ms": round(spp_ms, 4), "gflops": round(2.0 * d["nnz"] * K0 / (spp_ms * 1e6), 1), "runs": sp_info["spmm_runs"],
                          "alg_gbps": round(sp_bytes / (spp_ms * 1e6), 1), "hbm_frac": round(sp_bytes / (spp_ms * 1e6) / HBM_PEAK_GBPS, 4),
                          "max_diff_vs_csr_over_max": sp_diff, "plan_device_bytes": sp_info["device_bytes"]},
            "steps": n_steps}
        del x, y, Y
    if args.tile_sweep:
        # tile width x K slice x lanes per nonzero, explicit values honoured by the planner; fewer steps per row
        rows = []
        fit = {32: 1280, 64: 640, 128: 320}
        for ks in (32, 64, 128):
            if K0 % ks:
                continue
            for tx in sorted({fit[ks], fit[ks] // 2, 192}):
                if tx > fit[ks]:
                    continue
                for g in (4, 8):
                    try:
                        r = measure(K0, steps=max(10, args.steps // 10), warmup=max(3, args.warmup // 10), spinup=30.0,
                                    kernel=capi.KERNEL_LDS_TILE, tile_size_x=tx, k_slice=ks, tile_lanes=g)
                    except capi.SddmmError as e:
                        rows.append(dict(tile_size_x=tx, k_slice=ks, lanes_per_nnz=g, error=str(e)))
                        continue
                    i2 = r["info"]
                    rows.append(dict(tile_size_x=i2["tile_size_x"], tile_size_y=i2["tile_size_y"], k_slice=i2["k_slice"],
                                     lanes_per_nnz=i2["lanes_per_nnz"], n_col_tiles=i2["n_col_tiles"], lds_bytes=i2["lds_bytes"],
                                     grid=i2["grid"], block=i2["block"], padded_positions=i2["padded_positions"],
                                     ms=round(r["kernel_ms_mean"], 4), gflops=round(r["gflops"], 1),
                                     alg_gbps=round(r["alg_gbps"], 1), hbm_frac=round(r["frac"], 4)))
                    print("tile-sweep", rows[-1], file=sys.stderr, flush=True)
        line["tile_sweep"] = rows
    if not args.no_sweep and args.config == 3:
        sweep = {}
        for K in (32, 128, 256, 512):
            r = main_res if K == K0 else measure(K)
            sweep[str(K)] = {"gflops": round(r["gflops"], 1), "kernel_ms": round(r["kernel_ms_mean"], 4),
                             "hbm_frac": round(r["frac"], 4)}
        line["gflops_by_K"] = sweep
    # a plain 1 GiB copy kernel next to it (sddmm_copy_probe): with --copy-probe the known-size
    # reference the HBM counters of a profile are scaled by, always the bandwidth a streaming
    # kernel reaches on this device
    n = 1 << 30
    a = torch.empty(n // 4, device=dev); b = torch.empty_like(a)
    a.fill_(1.0)
    cs = torch.cuda.current_stream().cuda_stream
    capi.copy_probe(a.data_ptr(), b.data_ptr(), n, cs)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        capi.copy_probe(a.data_ptr(), b.data_ptr(), n, cs)
    e1.record()
    torch.cuda.synchronize()
    line["roofline"]["measured_copy_gbps"] = round(10 * 2.0 * n / (e0.elapsed_time(e1) * 1e6), 1)
    if args.copy_probe:
        line["copy_probe_bytes_each_way"] = n
    del a, b
    if not args.no_cpu:
        set_rank(K0)
        line["cpu_baseline"] = cpu_baseline(d, K0)
    if not args.no_sweep and not args.no_others and args.config == 3 and args.scale == 1.0 and not opt_fields:
        # The other benchmark shapes, each generated on the device, planned, spun up and timed like the main
        # one (the same steps and warm-up), with its own sample against the CPU oracle: the uniform plumbing
        # case, bag-of-words with the tile width the benchmark list states and with the planner's own, the
        # R-MAT graph, and the banded shape at both of its ranks.
        main_args = (args.tile_x, args.tile_y)
        others = []
        for cfg, K, tx in ((1, 32, 0), (2, 256, 192), (2, 256, 0), (4, 64, 0), (5, 512, 0), (5, 1024, 0)):
            d.clear()
            torch.cuda.empty_cache()
            t_gen = time.perf_counter()
            if not others or others[-1]["config"] != cfg:
                d2 = synth.make(cfg, 1.0, device=dev, K=K)
            torch.cuda.synchronize()
            t_gen = time.perf_counter() - t_gen
            args.tile_x, args.tile_y = tx, 0
            r = measure(K, keep_out=not args.no_parity, d=d2)
            i2 = r["info"]
            row = {"config": cfg, "workload": names[cfg], "n_rows": d2["n_rows"], "n_cols": d2["n_cols"], "nnz": d2["nnz"], "K": K,
                   "tile_size_x_asked": tx, "tile_size_x": i2["tile_size_x"], "tile_size_y": i2["tile_size_y"], "k_slice": i2["k_slice"],
                   "kernel": KERNEL_NAMES[i2["kernel"]], "kernel_launches_per_step": i2["n_launches"],
                   "ms_per_step": round(r["ms_per_step"], 5), "kernel_ms": round(r["kernel_ms_mean"], 5),
                   "graph_ms_per_step": round(r["graph_ms_per_step"], 5) if "graph_ms_per_step" in r else None,
                   "gflops": round(r["gflops"], 1), "alg_bytes_per_step": r["alg_bytes"], "alg_gbps": round(r["alg_gbps"], 1),
                   "hbm_frac": round(r["frac"], 4), "plan_ms": round(i2["plan_ms"], 1), "generate_s": round(t_gen, 2),
                   "kernels": [{"kernel": KERNEL_NAMES[p["kernel"]], "nnz": p["nnz"], "stream_positions": p["stream_positions"],
                                "launches": p["n_kernel_launches"], "ms": round(p["ms"], 5)} for p in r["prof"]]}
            tp = traffic_profile_path(cfg, 1.0, K, args.kernel, tx, 0, {})
            if tp:
                from sddmm_gpu_amd import rocprof
                row["traffic"] = rocprof.traffic_from_profile_text(tp)
                row["traffic_source"] = os.path.relpath(tp, ROOT) if row["traffic"] is not None else None
            if not args.no_parity:
                row["parity"] = parity_block(d2, K, r.pop("out"), torch)
            others.append(row)
            del r
            print("other-config", json.dumps(row), file=sys.stderr, flush=True)
        args.tile_x, args.tile_y = main_args
        del d2
        torch.cuda.empty_cache()
        line["other_configs"] = others
    line["config"]["executes"] = executes[0]
    line["config"]["argv"] = sys.argv[1:]
    if args.from_prof:
        from sddmm_gpu_amd import rocprof
        s = rocprof.summarize(args.from_prof)
        if s.get("traffic") is not None:
            line["roofline"]["traffic"] = s["traffic"]
            line["roofline"]["traffic_source"] = args.from_prof
        line["roofline"]["lds_bank_conflict_per_active"] = s.get("lds_bank_conflict_per_active")
        line["roofline"]["profile"] = {k: {f: e[f] for f in ("avg_us", "launches_per_step", "lds_bank_conflict_per_active",
                                                             "fma_share_of_valu") if f in e} for k, e in s["kernels"].items()}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
