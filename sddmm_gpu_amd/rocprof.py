"""Reads rocprofv3 CSV output of a bench.py run and turns it into the figures the
bench reports next to its timings: HBM bytes per SDDMM step (FETCH_SIZE /
WRITE_SIZE scaled by what the same counter reads for the copy probe, a plain copy
kernel of known size in the same run), LDS bank conflicts per active LDS cycle and
the average duration of every kernel.

A profile directory holds one sub-directory per rocprofv3 pass (the tool collects
one counter set per run), each with the pass's ``*_counter_collection.csv`` and/or
``*_kernel_trace.csv`` and, as ``run.json``, the JSON line the profiled bench run
printed (it carries ``config.executes``, the number of SDDMM steps the process
issued).  Typical passes, each a run of its own on the GPU box::

    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d DIR/fetch -o p -- \\
        python3 bench.py --no-cpu --no-sweep --steps 3 --warmup 1 --spinup-ms 0 --copy-probe > DIR/fetch/run.json
    (the same with WRITE_SIZE into DIR/write, and with
     SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_INSTS_VALU SQ_INSTS_VALU_FMA_F32 into DIR/lds)
    rocprofv3 --kernel-trace --stats --output-format csv -d DIR/stats -o p -- python3 bench.py ... > DIR/stats/run.json

``python -m sddmm_gpu_amd.rocprof DIR`` prints the summary as text (what is kept
under profiles/); ``bench.py --from-prof DIR`` merges it into the bench line.
"""
from __future__ import annotations

import collections
import csv
import json
import os
import re
import sys

PROBE = "sddmm_copy_probe_kernel"


def short_name(kernel_name: str) -> str:
    """'void (anonymous namespace)::sddmm_tile_kernel<8, 4, ...>(sddmm::TileArgs)' -> 'sddmm_tile_kernel<8,4,...>'"""
    m = re.search(r"(sddmm_[a-z_0-9]*kernel)(<[^>]*>)?", kernel_name)
    if not m:
        return kernel_name[:60]
    return m.group(1) + (m.group(2) or "").replace(" ", "")


def is_step_kernel(kernel_name: str) -> bool:
    """Kernels that sddmm_execute launches (not the probe, not the value re-ordering of set_values)."""
    return "sddmm_" in kernel_name and "kernel" in kernel_name and PROBE not in kernel_name


def _find(dirpath, suffix):
    out = []
    for base, _, files in os.walk(dirpath):
        out += [os.path.join(base, f) for f in files if f.endswith(suffix)]
    return sorted(out)


def read_pass(dirpath):
    """One rocprofv3 output directory -> dict(counters={(kernel, lds, grid): {counter: [per dispatch]}},
    durations={kernel: [ns]}, run=the bench line or None)."""
    counters = collections.defaultdict(lambda: collections.defaultdict(list))
    for path in _find(dirpath, "counter_collection.csv"):
        per_dispatch = collections.defaultdict(float)
        meta = {}
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                key = (r["Dispatch_Id"], r["Counter_Name"])
                per_dispatch[key] += float(r["Counter_Value"])
                meta[r["Dispatch_Id"]] = (r["Kernel_Name"], int(r.get("LDS_Block_Size") or 0), int(r.get("Grid_Size") or 0))
        for (disp, cname), v in per_dispatch.items():
            counters[meta[disp]][cname].append(v)
    durations = collections.defaultdict(list)
    for path in _find(dirpath, "kernel_trace.csv"):
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                durations[r["Kernel_Name"]].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    run = None
    p = os.path.join(dirpath, "run.json")
    if os.path.exists(p):
        for line in open(p):
            line = line.strip()
            if line.startswith("{"):
                run = json.loads(line)
    names = sorted({c for cs in counters.values() for c in cs})
    return dict(counters=counters, durations=durations, run=run, counter_names=names)


def summarize(profile_dir):
    """All passes under profile_dir -> one summary dict (see module docstring)."""
    passes = {}
    for name in sorted(os.listdir(profile_dir)):
        d = os.path.join(profile_dir, name)
        if os.path.isdir(d):
            passes[name] = read_pass(d)
    if not passes:
        passes["."] = read_pass(profile_dir)
    out = dict(profile_dir=profile_dir, passes=sorted(passes), kernels={}, traffic=None, notes=[], commands=[])
    kern = collections.defaultdict(dict)
    hbm = {}
    # passes without counters last: their kernel durations (undisturbed by counter collection) are the ones kept
    for pname, p in sorted(passes.items(), key=lambda kv: (not kv[1]["counter_names"], kv[0])):
        argv = (p["run"] or {}).get("config", {}).get("argv")
        pmc = ("--pmc " + " ".join(p["counter_names"]) + " ") if p["counter_names"] else "--stats "
        out["commands"].append(f"rocprofv3 {pmc}--kernel-trace --output-format csv -d {os.path.join(profile_dir, pname)} -o p -- "
                               f"python3 bench.py {' '.join(argv) if argv is not None else '<arguments not recorded>'}")
        executes = (p["run"] or {}).get("config", {}).get("executes")
        probe_bytes = (p["run"] or {}).get("copy_probe_bytes_each_way")
        # durations
        for k, ns in p["durations"].items():
            if is_step_kernel(k):
                e = kern[short_name(k)]
                e.setdefault("dispatches", len(ns))
                e["avg_us"] = round(sum(ns) / len(ns) / 1e3, 3)
                if executes:
                    e["launches_per_step"] = round(len(ns) / executes, 3)
        # counters
        for (k, lds, grid), cs in p["counters"].items():
            if not is_step_kernel(k):
                continue
            e = kern[short_name(k)]
            e["lds_bytes"] = lds
            e["grid_threads"] = grid
            for cname, vals in cs.items():
                e.setdefault("counters", {})[cname] = sum(vals) / len(vals)
        for cname in ("FETCH_SIZE", "WRITE_SIZE"):
            probe = [v for (k, _, _), cs in p["counters"].items() if PROBE in k for v in cs.get(cname, [])]
            step = [(short_name(k), v) for (k, _, _), cs in p["counters"].items() if is_step_kernel(k) for v in cs.get(cname, [])]
            if not step:
                continue
            if not probe or not probe_bytes or not executes:
                out["notes"].append(f"{pname}: {cname} present but no copy probe / run.json: not scaled")
                continue
            factor = (probe_bytes / 1024.0) / (sum(probe) / len(probe))  # counter is in KiB; the probe moves probe_bytes each way
            per_kernel = collections.defaultdict(float)
            for k, v in step:
                per_kernel[k] += v * 1024.0 * factor / executes
            hbm[cname] = dict(scale_factor=round(factor, 4), probe_kib=round(sum(probe) / len(probe), 1), executes=executes,
                              bytes_per_step=round(sum(per_kernel.values())),
                              by_kernel={k: round(v) for k, v in per_kernel.items()})
    for k, e in kern.items():
        c = e.get("counters", {})
        if c.get("SQ_LDS_IDX_ACTIVE"):
            e["lds_bank_conflict_per_active"] = round(c.get("SQ_LDS_BANK_CONFLICT", 0.0) / c["SQ_LDS_IDX_ACTIVE"], 5)
        if c.get("SQ_INSTS_VALU") and c.get("SQ_INSTS_VALU_FMA_F32") is not None:
            e["fma_share_of_valu"] = round(c["SQ_INSTS_VALU_FMA_F32"] / c["SQ_INSTS_VALU"], 4)
    out["kernels"] = dict(kern)
    out["hbm"] = hbm
    if "FETCH_SIZE" in hbm and "WRITE_SIZE" in hbm:
        out["traffic"] = hbm["FETCH_SIZE"]["bytes_per_step"] + hbm["WRITE_SIZE"]["bytes_per_step"]
    confl = [e["lds_bank_conflict_per_active"] for e in kern.values() if "lds_bank_conflict_per_active" in e]
    out["lds_bank_conflict_per_active"] = max(confl) if confl else None
    return out


def as_text(s):
    lines = [f"rocprofv3 summary of {s['profile_dir']} (passes: {', '.join(s['passes'])}), made by python3 -m sddmm_gpu_amd.rocprof {s['profile_dir']}",
             "each pass is a run of its own on the MI355X box, from the repository root, after cd /tmp && export TMPDIR=/tmp && cd back:"]
    lines += ["  " + c for c in s["commands"]]
    lines.append("(the line each run prints is kept as run.json in its pass directory: it carries the number of steps the run issued)")
    lines.append("(bytes per step = counter in KiB x 1024 x scale factor, summed over the kernels of one sddmm_execute; the scale factor is")
    lines.append(" the known size of the copy probe of the same run divided by what the counter reads for it)")
    for cname, h in s.get("hbm", {}).items():
        lines.append(f"{cname}: copy probe reads {h['probe_kib']} KiB -> scale factor {h['scale_factor']}; "
                     f"{h['executes']} steps in the run; bytes per step {h['bytes_per_step']:,}")
        for k, v in h["by_kernel"].items():
            lines.append(f"    {k:58s} {v:>16,} B per step")
    if s.get("traffic") is not None:
        lines.append(f"traffic_bytes_per_step: {s['traffic']}")
    if s.get("lds_bank_conflict_per_active") is not None:
        lines.append(f"lds_bank_conflict_per_active: {s['lds_bank_conflict_per_active']}")
    for k, e in s["kernels"].items():
        head = f"kernel {k}: " + ", ".join(f"{f}={e[f]}" for f in ("dispatches", "launches_per_step", "avg_us", "lds_bytes",
                                                                   "lds_bank_conflict_per_active", "fma_share_of_valu") if f in e)
        lines.append(head)
        for cname, v in sorted(e.get("counters", {}).items()):
            lines.append(f"    {cname:32s} {v:.6g} per dispatch")
    lines += ["note: " + n for n in s["notes"]]
    return "\n".join(lines)


def traffic_from_profile_text(path):
    """The 'traffic_bytes_per_step: N' line of a summary kept under profiles/ (None if absent)."""
    try:
        for line in open(path):
            m = re.match(r"traffic_bytes_per_step:\s*([0-9]+)", line)
            if m:
                return int(m.group(1))
    except OSError:
        pass
    return None


if __name__ == "__main__":
    if len(sys.argv) < 2:
        print(__doc__)
        sys.exit(2)
    print(as_text(summarize(sys.argv[1])))
