"""Full-size runs of the benchmark shapes on the GPU (generated there), checked
through properties that do not need a full CPU pass: a random sample of
nonzeros against the CPU oracle, exact power-of-two scaling, agreement of two
independent kernel families over every nonzero, and the pattern invariants
(sorted, duplicate-free, offsets consistent)."""
import numpy as np
import pytest
import torch

from conftest import parity_report, record_parity
from sddmm_gpu_amd import capi, synth

pytestmark = pytest.mark.gpu


def run(d, kernel, W=None, plan_values=False):
    dev = d["val"].device
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], d["row_ptr"].data_ptr(), d["col_ind"].data_ptr(),
                                     d["K"], 0, 0, kernel)
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    W = d["W"] if W is None else W
    stream = torch.cuda.current_stream().cuda_stream
    if plan_values:  # S.val handed to the plan once (what bench.py times) instead of passed per execute
        plan.set_values(d["val"].data_ptr(), stream)
    plan.execute(0 if plan_values else d["val"].data_ptr(), W.data_ptr(), d["H"].data_ptr(), out.data_ptr(), stream)
    torch.cuda.synchronize()
    info = plan.info()
    plan.close()
    return out, info


@pytest.mark.parametrize("cfg,K", [(3, 128), (3, 256), (3, 32), (3, 512), (4, 64), (5, 512), (5, 1024)])
def test_full_size(oracle, cfg, K):
    dev = torch.device("cuda:0")
    d = synth.make(cfg, 1.0, device=dev, K=K)
    n_rows, n_cols, nnz = d["n_rows"], d["n_cols"], d["nnz"]
    # pattern invariants: (row, col)-sorted, no duplicates, offsets match
    key = d["row_ind"].long() * n_cols + d["col_ind"].long()
    assert bool((key[1:] > key[:-1]).all())
    assert int(d["row_ptr"][-1]) == nnz and bool((d["row_ptr"][1:] >= d["row_ptr"][:-1]).all())
    assert torch.equal(torch.bincount(d["row_ind"].long(), minlength=n_rows), (d["row_ptr"][1:] - d["row_ptr"][:-1]).long())
    del key

    out, info = run(d, capi.KERNEL_AUTO)
    assert info["nnz"] == nnz and info["dense_nnz"] + sum(info["class_nnz"]) == nnz
    assert bool(torch.isfinite(out).all())

    # (1) a random sample of nonzeros against the CPU oracle
    g = torch.Generator(device=dev); g.manual_seed(99)
    idx = torch.randint(0, nnz, (400_000,), generator=g, device=dev)
    rows = d["row_ind"][idx].cpu().numpy(); cols = d["col_ind"][idx].cpu().numpy(); vals = d["val"][idx].cpu().numpy()
    W = d["W"].cpu().numpy(); H = d["H"].cpu().numpy()
    cpu = oracle.sddmm_coo(rows, cols, vals, W, H)
    f64, absp = oracle.sddmm_f64(rows, cols, vals, W, H)
    rep = parity_report(out[idx].cpu().numpy(), cpu, K, absp, f64=f64)
    record_parity(f"full size config {cfg} K={K} nnz={nnz} (sample of 400000)", rep)
    assert rep["violations"] == 0, rep
    assert rep["gpu_vs_f64_strict"] <= rep["cpu_vs_f64_strict"], rep
    del W, H

    # (1b) values kept by the plan in stream order: the same arithmetic, so the same bits
    outp, _ = run(d, capi.KERNEL_AUTO, plan_values=True)
    assert torch.equal(outp, out)
    del outp

    # (1c) the fused residual epilogue val - dot: the sample against the oracle (whose residual
    # form is val minus its scaled form with val = 1, bit for bit), and every nonzero against
    # val minus the GPU's own unscaled dot product (the same sums; only the last rounding and,
    # with K slices, the order of the subtractions differ)
    plan = capi.Plan.from_device_csr(n_rows, n_cols, nnz, d["row_ptr"].data_ptr(), d["col_ind"].data_ptr(), K, 0, 0,
                                     capi.KERNEL_AUTO)
    stream = torch.cuda.current_stream().cuda_stream
    dot = torch.empty(nnz, device=dev); res = torch.empty(nnz, device=dev)
    plan.execute(0, d["W"].data_ptr(), d["H"].data_ptr(), dot.data_ptr(), stream)            # no values: out = dot
    plan.execute_epilogue(d["val"].data_ptr(), d["W"].data_ptr(), d["H"].data_ptr(), res.data_ptr(),
                          capi.EPILOGUE_RESIDUAL, stream)
    torch.cuda.synchronize()
    plan.close()
    # (the partial dot products of the K slices can be larger than their sum: Cauchy-Schwarz bounds them)
    wn = torch.linalg.vector_norm(d["W"], dim=1); hn = torch.linalg.vector_norm(d["H"], dim=1)
    slack = 2.0 ** -22 * (d["val"].abs() + wn[d["row_ind"].long()] * hn[d["col_ind"].long()]) * max(1, K // 128)
    del wn, hn
    assert bool(((res - (d["val"] - dot)).abs() <= slack).all())
    W = d["W"].cpu().numpy(); H = d["H"].cpu().numpy()
    cpu_dot = oracle.sddmm_coo(rows, cols, np.ones_like(vals), W, H)
    _, absp1 = oracle.sddmm_f64(rows, cols, np.ones_like(vals), W, H)
    cpu_res = vals - cpu_dot
    lim = 1e-5 * np.sqrt(K) * np.maximum(np.abs(cpu_dot), absp1 / 100.0) + 2.0 ** -23 * np.abs(cpu_res)
    assert not (np.abs(res[idx].cpu().numpy().astype(np.float64) - cpu_res) > lim).any()
    del W, H, dot, res

    # (2) scaling W by a power of two scales every output exactly
    out4, _ = run(d, capi.KERNEL_AUTO, W=d["W"] * 4.0)
    assert torch.equal(out4, out * 4.0)
    del out4

    # (3) an independent kernel family agrees on every nonzero
    ref, rinfo = run(d, capi.KERNEL_ROW_GATHER)
    assert rinfo["kernel"] == capi.KERNEL_ROW_GATHER
    tol = 1e-5 * np.sqrt(K)
    # |val| * |W[r]|.|H[c]| >= |val| * sum|w h| / sqrt-free bound is costly; use the Cauchy-Schwarz bound instead
    wn = torch.linalg.vector_norm(d["W"], dim=1); hn = torch.linalg.vector_norm(d["H"], dim=1)
    bound = d["val"].abs() * wn[d["row_ind"].long()] * hn[d["col_ind"].long()]
    bad = (out - ref).abs() > tol * torch.maximum(ref.abs(), bound / 100.0)
    assert int(bad.sum()) == 0, (int(bad.sum()), float((out - ref).abs().max()))
