import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


PARITY_LOG = []  # (label, report) of every full comparison of this session, written out at its end


def record_parity(label, rep):
    PARITY_LOG.append((label, rep))


def pytest_sessionfinish(session, exitstatus):
    # the per-case figures (strict count, worst relative and norm-wise error, the oracle's own
    # strict count against fp64) as one JSON line per case, where a run's output is collected
    if not PARITY_LOG:
        return
    import json
    out = os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "parity_report.jsonl"), "w") as f:
            for label, rep in PARITY_LOG:
                f.write(json.dumps(dict(case=label, **rep)) + "\n")
    except OSError:
        pass


def parity_report(gpu, cpu, K, absdot=None, cond_limit=100.0, f64=None):
    """Compares GPU results with the CPU oracle's.

    The bar is |gpu - cpu| <= 1e-5*sqrt(K)*|cpu| per nonzero.  A dot product of
    signed terms can cancel to (almost) zero, and then no fp32 summation order
    agrees with another to a RELATIVE tolerance; for those nonzeros (condition
    number |val|*sum|w_t h_t| / |cpu| above cond_limit) the same tolerance is
    applied relative to |val|*sum|w_t h_t| / cond_limit instead.  Returns a dict
    with the worst errors and the number of violators of either form."""
    gpu = np.asarray(gpu, np.float64)
    cpu = np.asarray(cpu, np.float64)
    tol = 1e-5 * np.sqrt(K)
    diff = np.abs(gpu - cpu)
    strict_bad = diff > tol * np.abs(cpu)
    rep = dict(tol=tol, n=len(cpu), strict_violations=int(strict_bad.sum()),
               max_abs=float(diff.max()) if len(cpu) else 0.0)
    nz = np.abs(cpu) > 0
    rep["max_rel"] = float((diff[nz] / np.abs(cpu[nz])).max()) if nz.any() else 0.0
    if absdot is not None:
        absdot = np.asarray(absdot, np.float64)
        scale = np.maximum(np.abs(cpu), absdot / cond_limit)
        rep["violations"] = int((diff > tol * scale).sum())
        pos = absdot > 0
        rep["max_normwise"] = float((diff[pos] / absdot[pos]).max()) if pos.any() else 0.0
    else:
        rep["violations"] = rep["strict_violations"]
    if f64 is not None:
        # what fp32 summation order alone costs on this input: how many of the sequential CPU sums, and
        # how many of the GPU's, miss the strict bound against the fp64 value
        f64 = np.asarray(f64, np.float64)
        rep["cpu_vs_f64_strict"] = int((np.abs(cpu - f64) > tol * np.abs(f64)).sum())
        rep["gpu_vs_f64_strict"] = int((np.abs(gpu - f64) > tol * np.abs(f64)).sum())
    return rep


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o
