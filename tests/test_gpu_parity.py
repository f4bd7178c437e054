"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real
MI355X.  Pattern and output order are bit-exact by construction of the checks
(outputs are compared position by position with the oracle's, which runs on
the same sorted arrays); values must agree within 1e-5*sqrt(K) relative per
nonzero (see conftest.parity_report for nonzeros that cancel to ~0)."""
import numpy as np
import pytest
import torch

from conftest import parity_report, record_parity
from sddmm_gpu_amd import capi, synth

pytestmark = pytest.mark.gpu

KERNELS = {"row": capi.KERNEL_ROW_GATHER, "lds": capi.KERNEL_LDS_TILE, "panel": capi.KERNEL_PANEL,
           "hybrid": capi.KERNEL_HYBRID, "auto": capi.KERNEL_AUTO}


def plan_options(kernel=capi.KERNEL_AUTO, tile_x=0, tile_y=0, **fields):
    """The planner steered through sddmm_plan_options (the environment layer switched off)."""
    return capi.PlanOptions.defaults(ignore_env=1, kernel=kernel, tile_size_x=tile_x, tile_size_y=tile_y, **fields)


def run_gpu(d, K=None, tile_x=0, tile_y=0, kernel=capi.KERNEL_AUTO, use_plan_vals=True, opts=None):
    """d: dict from synth (CPU tensors); opts: fields of sddmm_plan_options.  Returns (out numpy, plan info)."""
    dev = torch.device("cuda:0")
    rows = d["row_ind"].numpy(); cols = d["col_ind"].numpy(); vals = d["val"].numpy()
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], rows, cols, vals)
    K = K or d["K"]
    plan = S.plan(K, tile_x, tile_y, kernel) if opts is None else S.plan(K, options=plan_options(kernel, tile_x, tile_y, **opts))
    W = d["W"].to(dev).contiguous(); H = d["H"].to(dev).contiguous()
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    dval = 0 if use_plan_vals else d["val"].to(dev)
    plan.execute(0 if use_plan_vals else dval.data_ptr(), W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    return out.cpu().numpy(), plan.info()


def check(d, out, oracle, K=None, label=None):
    """The bar of every comparison here.  Per nonzero: |gpu - cpu| <= 1e-5*sqrt(K)*|cpu|, or, where the
    terms of the dot product cancel (condition number above 100), the same tolerance against
    sum|w h|/100 -- no fp32 summation order meets a relative bound there, the sequential CPU sum
    included.  So that the relaxed form is not the only gate, the GPU's strict misses against the
    fp64 value must not outnumber the CPU oracle's own (both counts are in the report)."""
    K = K or d["K"]
    rows = d["row_ind"].numpy(); cols = d["col_ind"].numpy(); vals = d["val"].numpy()
    W = d["W"].numpy(); H = d["H"].numpy()
    cpu = oracle.sddmm_csr(d["row_ptr"].numpy(), cols, vals, W, H)
    assert np.array_equal(cpu, oracle.sddmm_coo(rows, cols, vals, W, H))
    f64, absp = oracle.sddmm_f64(rows, cols, vals, W, H)
    assert out.shape == cpu.shape and np.all(np.isfinite(out))
    rep = parity_report(out, cpu, K, absp, f64=f64)
    record_parity(label or f"{d.get('name', 'matrix')} {d['n_rows']}x{d['n_cols']} nnz={d['nnz']} K={K}", rep)
    assert rep["violations"] == 0, rep
    assert rep["gpu_vs_f64_strict"] <= rep["cpu_vs_f64_strict"], rep
    # the GPU's tree-shaped sum must not be less accurate than the sequential CPU sum
    err_gpu = np.abs(out - f64).max(); err_cpu = np.abs(cpu - f64).max()
    assert err_gpu <= 2 * err_cpu + 1e-30, (err_gpu, err_cpu, rep)
    return rep


@pytest.mark.parametrize("kernel", ["row", "lds", "panel"])
def test_config1_uniform_single_tile(oracle, kernel):
    d = synth.make(1)
    out, info = run_gpu(d, tile_x=4096, tile_y=4096, kernel=KERNELS[kernel])
    rep = check(d, out, oracle)
    assert info["nnz"] == d["nnz"] and info["K"] == 32
    if kernel == "lds":
        assert info["kernel"] == capi.KERNEL_LDS_TILE and info["tile_size_x"] <= 1280
    if kernel == "panel":
        assert info["kernel"] == capi.KERNEL_PANEL and info["k_slice"] == 32
    print(rep)


@pytest.mark.parametrize("kernel,tx,ty", [("auto", 192, 50000), ("row", 0, 0), ("lds", 64, 48), ("panel", 192, 50000), ("panel", 50, 100)])
def test_config2_bag_of_words(oracle, kernel, tx, ty):
    d = synth.make(2)
    out, info = run_gpu(d, tile_x=tx, tile_y=ty, kernel=KERNELS.get(kernel, capi.KERNEL_AUTO))
    rep = check(d, out, oracle)
    if kernel == "lds":
        assert info["kernel"] == capi.KERNEL_LDS_TILE and info["tile_size_x"] == 64
    if kernel == "auto":
        assert info["dense_nnz"] + sum(info["class_nnz"]) == d["nnz"] and sum(info["class_rows"]) == info["rows_touched"]
    print(info, rep)


@pytest.mark.parametrize("cfg,scale,K", [(3, 0.02, 128), (3, 0.02, 32), (3, 0.01, 256), (3, 0.005, 512),
                                         (4, 2.0 ** -7, 64), (5, 2.0 ** -6, 512), (5, 2.0 ** -7, 1024)])
@pytest.mark.parametrize("kernel", ["row", "lds", "panel", "auto"])
def test_scaled_configs(oracle, cfg, scale, K, kernel):
    d = synth.make(cfg, scale, K=K)
    out, info = run_gpu(d, kernel=KERNELS[kernel])
    check(d, out, oracle)


@pytest.mark.parametrize("K", [1, 3, 4, 20, 36, 96, 100, 192, 384, 2048, 2052])
def test_odd_ranks(oracle, K):
    d = synth.uniform_random(300, 500, 0.05, K=K, seed=40 + K)
    for kernel in ("row", "lds", "panel"):
        out, info = run_gpu(d, tile_x=64, kernel=KERNELS[kernel])
        check(d, out, oracle)
        if kernel == "panel":
            assert info["kernel"] == (capi.KERNEL_PANEL if K % 32 == 0 else capi.KERNEL_ROW_GATHER)


def test_edge_shapes(oracle):
    rng = np.random.default_rng(7)
    K = 64
    cases = {
        "single_nonzero": ([5], [7]),
        "one_full_row": (np.full(300, 3), np.arange(300)),
        "one_full_col": (np.arange(200), np.full(200, 11)),
        "diag": (np.arange(150), np.arange(150)),
        "first_and_last": ([0, 299], [0, 299]),
        "exactly_64": (np.repeat(np.arange(8), 8), np.tile(np.arange(8), 8)),
        "exactly_65": (np.concatenate([np.repeat(np.arange(8), 8), [9]]), np.concatenate([np.tile(np.arange(8), 8), [0]])),
    }
    for name, (r, c) in cases.items():
        r = np.asarray(r, np.int32); c = np.asarray(c, np.int32)
        n, m = 300, 300
        d = dict(n_rows=n, n_cols=m, nnz=len(r), K=K, row_ind=torch.from_numpy(r), col_ind=torch.from_numpy(c),
                 row_ptr=torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(r, minlength=n))]).astype(np.int32)),
                 val=torch.from_numpy(rng.standard_normal(len(r)).astype(np.float32)),
                 W=torch.from_numpy(rng.standard_normal((n, K)).astype(np.float32)),
                 H=torch.from_numpy(rng.standard_normal((m, K)).astype(np.float32)))
        for kernel, tx, ty in (("row", 0, 0), ("lds", 7, 3), ("lds", 300, 1), ("panel", 7, 3), ("panel", 0, 0)):
            out, info = run_gpu(d, tile_x=tx, tile_y=ty, kernel=KERNELS[kernel])
            check(d, out, oracle)


def _dict_of(n, m, r, c, K, rng):
    r = np.asarray(r, np.int32); c = np.asarray(c, np.int32)
    order = np.lexsort((c, r)); r = r[order]; c = c[order]
    return dict(n_rows=n, n_cols=m, nnz=len(r), K=K, row_ind=torch.from_numpy(r), col_ind=torch.from_numpy(c),
                row_ptr=torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(r, minlength=n))]).astype(np.int32)),
                val=torch.from_numpy(rng.standard_normal(len(r)).astype(np.float32)),
                W=torch.from_numpy(rng.standard_normal((n, K)).astype(np.float32)),
                H=torch.from_numpy(rng.standard_normal((m, K)).astype(np.float32)))


@pytest.mark.parametrize("forced", [False, True])
def test_extreme_shapes_through_the_planner(oracle, forced):
    """Degenerate shapes through AUTO and HYBRID, once with the planner's own choices
    and once with its size thresholds removed, so that the tiled and split plans (and
    their short batches) are built for inputs they would normally never see."""
    opts = dict(split_min_nnz=0, stage_factor=0) if forced else None
    rng = np.random.default_rng(123)
    wide = np.unique(rng.integers(0, 150000, 60000))
    cases = [
        ("one_by_one", 1, 1, [0], [0], 128),
        ("one_long_row", 1, 150000, np.zeros(len(wide)), wide, 128),
        ("one_long_col", 150000, 1, wide, np.zeros(len(wide)), 128),
        ("one_row_of_three", 3, 700, [1, 1, 1], [0, 350, 699], 128),
        ("dense_block", 96, 640, np.repeat(np.arange(96), 640), np.tile(np.arange(640), 96), 128),
        ("dense_block_k256", 64, 300, np.repeat(np.arange(64), 300), np.tile(np.arange(300), 64), 256),
        ("runs_of_1_to_9", 45, 600, np.repeat(np.arange(45), np.arange(45) % 9 + 1),
         np.concatenate([np.arange(k % 9 + 1) * 7 + k for k in range(45)]), 128),
        ("rank_4", 500, 400, *np.divmod(np.unique(rng.integers(0, 500 * 400, 9000)), 400), 4),
        ("rank_8", 500, 400, *np.divmod(np.unique(rng.integers(0, 500 * 400, 9000)), 400), 8),
        ("rank_1024", 120, 90, *np.divmod(np.unique(rng.integers(0, 120 * 90, 3000)), 90), 1024),
        ("rank_2048", 60, 50, *np.divmod(np.unique(rng.integers(0, 60 * 50, 900)), 50), 2048),
    ]
    for name, n, m, r, c, K in cases:
        d = _dict_of(n, m, r, c, K, rng)
        for kernel in ("auto", "hybrid"):
            out, info = run_gpu(d, kernel=KERNELS[kernel], opts=opts)
            rep = check(d, out, oracle)
            assert info["dense_nnz"] + sum(info["class_nnz"]) == d["nnz"], (name, kernel, info)


def test_empty_matrix_and_empty_rows(oracle):
    S = capi.Coo.from_arrays(10, 10, [], [])
    plan = S.plan(32)
    plan.execute(0, 0, 0, 0)  # nnz == 0: nothing is touched
    assert plan.info()["nnz"] == 0
    d = synth.uniform_random(2000, 100, 0.002, K=32, seed=9)  # most rows empty
    assert (np.diff(d["row_ptr"].numpy()) == 0).mean() > 0.5
    for kernel in ("row", "lds", "panel"):
        out, _ = run_gpu(d, tile_x=16, tile_y=5, kernel=KERNELS[kernel])
        check(d, out, oracle)


def test_closed_forms_on_gpu():
    d = synth.make(1)
    dev = torch.device("cuda:0")
    for kernel in ("row", "lds", "panel"):
        for K in (32, 100, 7):
            S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
            plan = S.plan(K, 256, 64, KERNELS[kernel])
            W = torch.ones(d["n_rows"], K, device=dev); H = torch.ones(d["n_cols"], K, device=dev)
            out = torch.empty(d["nnz"], device=dev)
            plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
            assert torch.equal(out.cpu(), d["val"] * K)            # W = H = 1  ->  K * val
            j = torch.randint(0, K, (d["n_cols"],), generator=torch.Generator().manual_seed(1))
            Hoh = torch.zeros(d["n_cols"], K); Hoh[torch.arange(d["n_cols"]), j] = 1.0
            Wr = torch.randn(d["n_rows"], K, generator=torch.Generator().manual_seed(2))
            Wd = Wr.to(dev); Hd = Hoh.to(dev)
            plan.execute(0, Wd.data_ptr(), Hd.data_ptr(), out.data_ptr())
            expect = Wr[d["row_ind"].long(), j[d["col_ind"].long()]] * d["val"]
            assert torch.equal(out.cpu(), expect)                  # one-hot H picks W[r, j(c)]


def test_value_sources_and_host_form(oracle):
    d = synth.make(3, 0.01, K=64)
    rows = d["row_ind"].numpy(); cols = d["col_ind"].numpy(); vals = d["val"].numpy()
    W = d["W"].numpy(); H = d["H"].numpy()
    dev = torch.device("cuda:0")
    # (a) values passed at execute override the plan's
    out_a, _ = run_gpu(d, use_plan_vals=False)
    check(d, out_a, oracle)
    # (b) a plan over a device-resident CSR, no values: out = dot (the shipping reference's form)
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev)
    for kernel in (capi.KERNEL_ROW_GATHER, capi.KERNEL_LDS_TILE, capi.KERNEL_PANEL):
        plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), 64, 128, 32,
                                         kernel, keep=(rp, ci))
        Wd = d["W"].to(dev); Hd = d["H"].to(dev); out = torch.empty(d["nnz"], device=dev)
        plan.execute(0, Wd.data_ptr(), Hd.data_ptr(), out.data_ptr())
        cpu = oracle.sddmm_coo(rows, cols, vals, W, H, apply_val=False)
        _, absp = oracle.sddmm_f64(rows, cols, np.ones_like(vals), W, H)
        assert parity_report(out.cpu().numpy(), cpu, 64, absp)["violations"] == 0
        dv = d["val"].to(dev)
        plan.execute(dv.data_ptr(), Wd.data_ptr(), Hd.data_ptr(), out.data_ptr())
        check(d, out.cpu().numpy(), oracle)
        # values handed to the plan once, then changed: execute(NULL) must follow them
        plan.set_values(dv.data_ptr())
        plan.execute(0, Wd.data_ptr(), Hd.data_ptr(), out.data_ptr())
        check(d, out.cpu().numpy(), oracle)
        dv2 = dv * 2.0
        plan.set_values(dv2.data_ptr())
        plan.execute(0, Wd.data_ptr(), Hd.data_ptr(), out.data_ptr())
        d2 = dict(d); d2["val"] = d["val"] * 2.0
        check(d2, out.cpu().numpy(), oracle)
    # the same on a hybrid plan with both row classes, built from the options structure
    opts = capi.PlanOptions.defaults(kernel=capi.KERNEL_HYBRID, short_row_max=15, split_min_nnz=0, stage_factor=0, ignore_env=1)
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), 64, keep=(rp, ci),
                                     options=opts)
    assert plan.info()["class_nnz"][0] > 0 and plan.info()["class_nnz"][2] > 0
    i_ = plan.info(); assert i_["dense_nnz"] + sum(i_["class_nnz"]) == d["nnz"]
    plan.set_values(dv.data_ptr())
    plan.execute(0, Wd.data_ptr(), Hd.data_ptr(), out.data_ptr())
    check(d, out.cpu().numpy(), oracle)
    # (c) host-pointer form with the reference's sddmm_GPU convention
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], rows, cols, vals)
    out_c, ms = S.plan(64).gpu(W, H)
    check(d, out_c, oracle)
    assert ms > 0


def residual_ok(out, d, oracle, K):
    """|gpu - cpu| of val - dot within the tolerance of the dot product (the error is
    the dot product's) plus one rounding of the subtraction."""
    rows = d["row_ind"].numpy(); cols = d["col_ind"].numpy(); vals = d["val"].numpy()
    W = d["W"].numpy(); H = d["H"].numpy()
    cpu = oracle.sddmm_residual_csr(d["row_ptr"].numpy(), cols, vals, W, H)
    dot = oracle.sddmm_csr(d["row_ptr"].numpy(), cols, np.ones_like(vals), W, H)
    _, absp = oracle.sddmm_f64(rows, cols, np.ones_like(vals), W, H)
    tol = 1e-5 * np.sqrt(K)
    bound = tol * np.maximum(np.abs(dot), absp / 100.0) + 2.0 ** -23 * np.abs(cpu)
    assert out.shape == cpu.shape and np.all(np.isfinite(out))
    bad = np.abs(out.astype(np.float64) - cpu) > bound
    assert not bad.any(), (int(bad.sum()), float(np.abs(out - cpu).max()))


@pytest.mark.parametrize("kernel,K", [("row", 32), ("row", 100), ("row", 30), ("lds", 64), ("lds", 100), ("panel", 128),
                                      ("panel", 512), ("auto", 32), ("auto", 64), ("auto", 128), ("auto", 256), ("auto", 512)])
def test_residual_epilogue(oracle, kernel, K):
    """out = val - dot fused into every kernel family's store, with the values owned
    by the plan (stream order) and passed at execute (sorted order), in one K slice
    and in several; the scaled form through the same entry point gives sddmm_execute's bits."""
    d = synth.make(3, 0.05, K=K, seed=21)
    dev = torch.device("cuda:0")
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    plan = S.plan(K, options=plan_options(KERNELS[kernel], split_min_nnz=0))
    W = d["W"].to(dev); H = d["H"].to(dev); dv = d["val"].to(dev)
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute_epilogue(0, W.data_ptr(), H.data_ptr(), out.data_ptr(), capi.EPILOGUE_RESIDUAL)
    torch.cuda.synchronize()
    residual_ok(out.cpu().numpy(), d, oracle, K)
    out2 = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute_epilogue(dv.data_ptr(), W.data_ptr(), H.data_ptr(), out2.data_ptr(), capi.EPILOGUE_RESIDUAL)
    torch.cuda.synchronize()
    residual_ok(out2.cpu().numpy(), d, oracle, K)
    a = torch.empty(d["nnz"], device=dev); b = torch.empty(d["nnz"], device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), a.data_ptr())
    plan.execute_epilogue(0, W.data_ptr(), H.data_ptr(), b.data_ptr(), capi.EPILOGUE_SCALE)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_residual_epilogue_needs_values():
    d = synth.make(1, 0.25)
    dev = torch.device("cuda:0")
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev)
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), d["K"], 0, 0,
                                     capi.KERNEL_AUTO, keep=(rp, ci))
    W = d["W"].to(dev); H = d["H"].to(dev); out = torch.empty(d["nnz"], device=dev)
    with pytest.raises(capi.SddmmError) as e:
        plan.execute_epilogue(0, W.data_ptr(), H.data_ptr(), out.data_ptr(), capi.EPILOGUE_RESIDUAL)
    assert e.value.code == capi.ERR_ARG
    with pytest.raises(capi.SddmmError) as e:
        plan.execute_epilogue(0, W.data_ptr(), H.data_ptr(), out.data_ptr(), 7)
    assert e.value.code == capi.ERR_ARG


@pytest.mark.parametrize("K", [64, 256])
def test_execute_can_be_captured_in_a_graph(oracle, K):
    """sddmm_execute only launches kernels on the caller's stream (no allocation, no
    memset, no synchronisation), so a caller may record it into a HIP graph.  The graph
    is replayed several times with eager work and synchronisations in between and with
    W changed in place; every replay must give the eager result's bits."""
    d = synth.make(3, 0.05, K=K, seed=31)
    dev = torch.device("cuda:0")
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    plan = S.plan(K, options=plan_options(split_min_nnz=0))  # the split plan: two launches per K slice
    W = d["W"].to(dev).contiguous(); H = d["H"].to(dev).contiguous()
    out = torch.zeros(d["nnz"], device=dev); eager = torch.zeros(d["nnz"], device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr(), side.cuda_stream)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        W.mul_(2.0 if rep else 1.0)          # eager work between the replays
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        plan.execute(0, W.data_ptr(), H.data_ptr(), eager.data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
    d2 = dict(d); d2["W"] = d["W"] * 4.0
    check(d2, out.cpu().numpy(), oracle, K=K)


def test_device_plan_rejects_bad_csr():
    dev = torch.device("cuda:0")
    rp = torch.tensor([0, 2, 3], dtype=torch.int32, device=dev)
    bad_sorted = torch.tensor([5, 1, 0], dtype=torch.int32, device=dev)
    with pytest.raises(capi.SddmmError) as e:
        capi.Plan.from_device_csr(2, 8, 3, rp.data_ptr(), bad_sorted.data_ptr(), 32)
    assert e.value.code == capi.ERR_UNSORTED
    bad_range = torch.tensor([1, 9, 0], dtype=torch.int32, device=dev)
    with pytest.raises(capi.SddmmError) as e:
        capi.Plan.from_device_csr(2, 8, 3, rp.data_ptr(), bad_range.data_ptr(), 32)
    assert e.value.code == capi.ERR_RANGE


def test_power_of_two_scaling_is_exact_and_tilings_agree(oracle):
    d = synth.make(2)
    base, _ = run_gpu(d, kernel=capi.KERNEL_ROW_GATHER)
    d2 = dict(d); d2["W"] = d["W"] * 4.0
    out4, _ = run_gpu(d2, kernel=capi.KERNEL_ROW_GATHER)
    assert np.array_equal(out4, base * 4.0)
    _, absp = oracle.sddmm_f64(d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy(), d["W"].numpy(), d["H"].numpy())
    for kernel in (capi.KERNEL_LDS_TILE, capi.KERNEL_PANEL):
        for tx, ty in ((160, 50000), (50, 10), (1, 1), (12419, 1500)):
            out, info = run_gpu(d, tile_x=tx, tile_y=ty, kernel=kernel)
            assert parity_report(out, base, d["K"], absp)["violations"] == 0, (kernel, tx, ty)


@pytest.mark.parametrize("short_max", [20, 100, 10 ** 9, 0])
def test_hybrid_row_classes(oracle, short_max):
    """Forces the two row classes of a hybrid plan (long: tile kernel, short: padded
    gather) through the length threshold and checks the union of their outputs."""
    d = synth.make(3, 0.02, K=128)
    deg = np.diff(d["row_ptr"].numpy())
    # (split even this small matrix)
    out, info = run_gpu(d, tile_x=100, kernel=capi.KERNEL_HYBRID, opts=dict(short_row_max=short_max, split_min_nnz=0, stage_factor=0))
    check(d, out, oracle)
    assert info["dense_nnz"] + sum(info["class_nnz"]) == d["nnz"]
    assert sum(info["class_rows"]) == int((deg > 0).sum())
    if short_max == 20:
        assert info["kernel"] == capi.KERNEL_HYBRID and info["n_launches"] == 2
        assert info["class_rows"][0] == int((deg >= 20).sum())


@pytest.mark.parametrize("K,opts", [
    (64, {}), (192, {}), (256, {}), (512, {}),
    (128, dict(tile_waves=16)),                             # 16 instead of 12 waves per workgroup
    (128, dict(tile_assign=1)), (128, dict(tile_assign=0)),  # other work assignments
    (256, dict(k_slice=256)),                               # one full-K slice: variant G=16, 4 float4 per lane
    (512, dict(k_slice=256, dense_blocks=0)),               # two slices of 256
    (512, dict(k_slice=512, dense_blocks=0)),               # variant G=16 or 32
    (128, dict(tile_lanes=4)),                              # groups of 4 lanes in the tile kernel
    (128, dict(gather_lanes=4)), (256, dict(gather_padded=0)),
])
def test_hybrid_plan_ranks_and_variants(oracle, K, opts):
    """The split plan (tile kernel + padded gather) at several ranks and with the
    planner's alternatives forced through the options."""
    opts = dict(opts, split_min_nnz=0)
    d = synth.make(3, 0.06, K=K, seed=77)
    out, info = run_gpu(d, kernel=capi.KERNEL_AUTO, opts=opts)
    check(d, out, oracle)
    assert info["dense_nnz"] + sum(info["class_nnz"]) == d["nnz"]
    assert info["kernel"] == capi.KERNEL_HYBRID and info["class_nnz"][0] + info["dense_nnz"] > 0 and info["class_nnz"][2] > 0, info
    # the same plan with the values handed over once must give the same bits
    dev = torch.device("cuda:0")
    dd = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in d.items()}
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], dd["row_ptr"].data_ptr(), dd["col_ind"].data_ptr(),
                                     K, options=plan_options(**opts))
    plan.set_values(dd["val"].data_ptr())
    out2 = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(0, dd["W"].data_ptr(), dd["H"].data_ptr(), out2.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(out2.cpu().numpy(), out)


@pytest.mark.parametrize("K,opts", [(128, {}), (256, {}), (512, {}), (128, dict(tile_waves=16))])
def test_short_batches(oracle, K, opts):
    """Run ends with at most four nonzeros are collected, eight to a batch, into
    batches that the tile kernel runs in half the steps (both halves of a group of
    eight lanes then hold the same nonzeros).  The plan must report such batches, the
    results must stay within the tolerance of the oracle, two executes must give the
    same bits (the duplicate positions store the same value to the same place), and
    with the switch off there are none."""
    opts = dict(opts, split_min_nnz=0)
    d = synth.make(3, 0.06, K=K, seed=5)
    out, info = run_gpu(d, kernel=capi.KERNEL_AUTO, opts=opts)
    check(d, out, oracle)
    assert info["short_batches"] > 0 and info["short_batches"] * 64 < info["padded_positions"], info
    out_again, _ = run_gpu(d, kernel=capi.KERNEL_AUTO, opts=opts)
    assert np.array_equal(out, out_again)
    out_off, info_off = run_gpu(d, kernel=capi.KERNEL_AUTO, opts=dict(opts, tile_short_batches=0))
    check(d, out_off, oracle)
    assert info_off["short_batches"] == 0 and info_off["padded_positions"] <= info["padded_positions"]


@pytest.mark.parametrize("seed", list(range(48)))
def test_random_shapes_kernels_and_tilings(oracle, seed):
    """Seeded random shapes, densities, ranks, kernels and tile sizes; every second
    case lets the planner split even a small matrix into its row classes."""
    rng = np.random.default_rng(1000 + seed)
    n_rows = int(rng.integers(1, 3000)); n_cols = int(rng.integers(1, 6000))
    K = int(rng.choice([4, 8, 12, 32, 64, 96, 128, 256, 512]))
    kernel = str(rng.choice(["auto", "row", "lds", "hybrid", "panel"]))
    tile_x = int(rng.choice([0, 1, 7, 64, 192, 320, 5000])); tile_y = int(rng.choice([0, 1, 33, 50000]))
    opts = None
    if seed % 2:
        rng.integers(2, 200)  # (keeps the random stream of the cases that follow)
        # (tile even where staging the H tiles does not pay)
        opts = dict(split_min_nnz=0, stage_factor=0, short_row_max=int(rng.integers(1, 40)))
    # rows of very unequal length: a few long ones, many short or empty ones
    deg = np.minimum(n_cols, (rng.pareto(1.2, n_rows) * rng.integers(1, 30)).astype(np.int64))
    deg[rng.random(n_rows) < 0.2] = 0
    rows = np.repeat(np.arange(n_rows, dtype=np.int64), deg)
    cols = rng.integers(0, n_cols, len(rows))
    key = np.unique(rows * n_cols + cols)
    if len(key) == 0:
        key = np.array([0], dtype=np.int64)
    r = (key // n_cols).astype(np.int32); c = (key % n_cols).astype(np.int32)
    d = dict(n_rows=n_rows, n_cols=n_cols, nnz=len(r), K=K, row_ind=torch.from_numpy(r), col_ind=torch.from_numpy(c),
             row_ptr=torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(r, minlength=n_rows))]).astype(np.int32)),
             val=torch.from_numpy(rng.standard_normal(len(r)).astype(np.float32)),
             W=torch.from_numpy(rng.standard_normal((n_rows, K)).astype(np.float32)),
             H=torch.from_numpy(rng.standard_normal((n_cols, K)).astype(np.float32)))
    out, info = run_gpu(d, tile_x=tile_x, tile_y=tile_y, kernel=KERNELS[kernel], opts=opts)
    rows_np = d["row_ind"].numpy(); cols_np = d["col_ind"].numpy(); vals = d["val"].numpy()
    cpu = oracle.sddmm_csr(d["row_ptr"].numpy(), cols_np, vals, d["W"].numpy(), d["H"].numpy())
    _, absp = oracle.sddmm_f64(rows_np, cols_np, vals, d["W"].numpy(), d["H"].numpy())
    rep = parity_report(out, cpu, K, absp)
    assert rep["violations"] == 0, (rep, n_rows, n_cols, K, kernel, tile_x, tile_y, info)
    assert info["dense_nnz"] + sum(info["class_nnz"]) == d["nnz"]
