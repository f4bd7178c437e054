"""Plans built from the options structure (sddmm_plan_create_opt): the same plan as
the environment override layer gives, the unpadded and sub-list launches after
sddmm_plan_set_values, and the dense-block launch on the matrix cores in every value
mode and epilogue."""
import numpy as np
import pytest
import torch

from conftest import parity_report
from sddmm_gpu_amd import capi, synth
from test_gpu_parity import check, residual_ok

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def host_plan(d, K, **opt):
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    return S.plan(K, options=capi.PlanOptions.defaults(ignore_env=1, **opt))


def test_options_equal_environment_overrides(monkeypatch):
    d = synth.make(3, 0.05, K=128, seed=5)
    a = host_plan(d, 128, split_min_nnz=0, short_row_max=40, tile_short_batches=0)
    monkeypatch.setenv("SDDMM_SPLIT_MIN_NNZ", "0")
    monkeypatch.setenv("SDDMM_SHORT_ROW_MAX", "40")
    monkeypatch.setenv("SDDMM_TILE_SHORT", "0")
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    b = S.plan(128)
    ia, ib = a.info(), b.info()
    for k in ia:
        if k != "plan_ms":
            assert ia[k] == ib[k], k
    ob = b.options()
    assert ob["split_min_nnz"] == 0 and ob["short_row_max"] == 40 and ob["tile_short_batches"] == 0  # reported back
    # ignore_env: the same call with the variables still set builds the default plan
    c = S.plan(128, options=capi.PlanOptions.defaults(ignore_env=1))
    assert c.options()["short_row_max"] == -1
    dev = torch.device(DEV)
    W = d["W"].to(dev); H = d["H"].to(dev)
    oa = torch.empty(d["nnz"], device=dev); ob_ = torch.empty(d["nnz"], device=dev)
    a.execute(0, W.data_ptr(), H.data_ptr(), oa.data_ptr())
    b.execute(0, W.data_ptr(), H.data_ptr(), ob_.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(oa, ob_)


@pytest.mark.parametrize("K", [96, 100])
def test_set_values_reaches_the_unpadded_lds_tile_launch(oracle, K):
    # a K without a padded tile variant: the LDS_TILE plan is the unpadded stream kernel, which
    # keeps its own stream-order copy of the values
    d = synth.uniform_random(700, 900, 0.03, K=K, seed=70 + K)
    plan = host_plan(d, K, kernel=capi.KERNEL_LDS_TILE, tile_size_x=64, unpadded_tile=1)
    assert plan.info()["kernel"] == capi.KERNEL_LDS_TILE
    dev = torch.device(DEV)
    W = d["W"].to(dev); H = d["H"].to(dev); out = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    check(d, out.cpu().numpy(), oracle, K)
    dv2 = (d["val"] * 2.0 + 1.0).to(dev)
    plan.set_values(dv2.data_ptr())
    plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    d2 = dict(d); d2["val"] = d["val"] * 2.0 + 1.0
    check(d2, out.cpu().numpy(), oracle, K)


def test_set_values_reaches_the_row_gather_sublist_launch(oracle):
    # hybrid plan whose short class is the plain row gather over a list of rows (its own permuted stream)
    K = 64
    d = synth.make(3, 0.02, K=K, seed=8)
    plan = host_plan(d, K, kernel=capi.KERNEL_HYBRID, split_min_nnz=0, short_row_max=30, gather_padded=0, stage_factor=0)
    info = plan.info()
    assert info["class_nnz"][0] > 0 and info["class_nnz"][2] > 0
    dev = torch.device(DEV)
    W = d["W"].to(dev); H = d["H"].to(dev); out = torch.full((d["nnz"],), float("nan"), device=dev)
    dv2 = (d["val"] * 0.5 - 3.0).to(dev)
    plan.set_values(dv2.data_ptr())
    plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    d2 = dict(d); d2["val"] = d["val"] * 0.5 - 3.0
    check(d2, out.cpu().numpy(), oracle, K)


@pytest.mark.parametrize("cfg,scale,K", [(3, 0.06, 128), (2, 1.0, 256), (3, 0.03, 512), (3, 0.03, 32)])
def test_dense_block_launch(oracle, cfg, scale, K):
    """The dense core on the matrix cores (fp32 MFMA), the remainder through the tile and gather
    launches: no values, values at execute, values owned by the plan, and the residual epilogue."""
    d = synth.make(cfg, scale, K=K)
    dev = torch.device(DEV)
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev)
    opts = capi.PlanOptions.defaults(kernel=capi.KERNEL_HYBRID, dense_blocks=1, dense_min_nnz=1000, split_min_nnz=0, ignore_env=1)
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), K, keep=(rp, ci),
                                     options=opts)
    info = plan.info()
    if K == 32:
        assert info["dense_nnz"] == 0  # (the compact tile stream of narrow slices cannot address a remainder)
    else:
        assert info["dense_nnz"] > d["nnz"] // 10 and info["dense_blocks"] > 0, info
    assert info["dense_nnz"] + sum(info["class_nnz"]) == d["nnz"]
    W = d["W"].to(dev); H = d["H"].to(dev); dv = d["val"].to(dev)
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    rows = d["row_ind"].numpy(); cols = d["col_ind"].numpy(); vals = d["val"].numpy()
    plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    cpu1 = oracle.sddmm_coo(rows, cols, vals, d["W"].numpy(), d["H"].numpy(), apply_val=False)
    _, absp1 = oracle.sddmm_f64(rows, cols, np.ones_like(vals), d["W"].numpy(), d["H"].numpy())
    assert parity_report(out.cpu().numpy(), cpu1, K, absp1)["violations"] == 0
    out.fill_(float("nan"))
    plan.execute(dv.data_ptr(), W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    check(d, out.cpu().numpy(), oracle, K)
    plan.set_values(dv.data_ptr())
    out2 = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), out2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    for src in (0, dv.data_ptr()):
        out.fill_(float("nan"))
        plan.execute_epilogue(src, W.data_ptr(), H.data_ptr(), out.data_ptr(), capi.EPILOGUE_RESIDUAL)
        torch.cuda.synchronize()
        residual_ok(out.cpu().numpy(), d, oracle, K)


@pytest.mark.parametrize("K,slab,panel", [(64, 4096, -1), (64, 1000, 3000), (128, 2048, -1), (256, 512, -1), (32, 8192, 100)])
def test_padded_gather_over_column_slabs(oracle, K, slab, panel):
    """The padded gather walking S slab by slab (and row panel by row panel), the form AUTO builds when H is far
    larger than the caches: same results as the oracle, values in every mode."""
    d = synth.make(4, 2.0 ** -7, K=K)
    dev = torch.device(DEV)
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev); dv = d["val"].to(dev)
    opts = capi.PlanOptions.defaults(kernel=capi.KERNEL_ROW_GATHER, row_padded=1, gather_lanes=4 if K <= 128 else 8,
                                     gather_slab_cols=slab, gather_panel_rows=panel, ignore_env=1)
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), K, keep=(rp, ci), options=opts)
    info = plan.info()
    assert info["padded_positions"] >= d["nnz"]
    W = d["W"].to(dev); H = d["H"].to(dev)
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(dv.data_ptr(), W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    check(d, out.cpu().numpy(), oracle, K)
    plan.set_values(dv.data_ptr())
    out2 = torch.full_like(out, float("nan"))
    plan.execute(0, W.data_ptr(), H.data_ptr(), out2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    out2.fill_(float("nan"))
    plan.execute_epilogue(0, W.data_ptr(), H.data_ptr(), out2.data_ptr(), capi.EPILOGUE_RESIDUAL)
    torch.cuda.synchronize()
    residual_ok(out2.cpu().numpy(), d, oracle, K)


@pytest.mark.parametrize("K", [128, 256])
def test_banded_rows_walked_by_groups_of_workgroups(oracle, tmp_path, K):
    """More column tiles than workgroups and rows that touch a dozen tiles each: the rows are cut into ranges, each
    walked by a group of workgroups of one die (tile_runs = 2).  Checked against the oracle like the plan with whole
    tiles handed out in runs of neighbours (tile_runs = 1); the two differ in the last bits where a run's short last
    chunk lands in a batch of the other kind (the items end elsewhere), never by more than a few ulps of the sum."""
    d = synth.banded(n=16384, per_row=24, half_band=96, K=K, seed=21)
    outs = {}
    for runs in (1, 2):
        plan = host_plan(d, K, kernel=capi.KERNEL_LDS_TILE, tile_size_x=16, tile_runs=runs)
        info = plan.info()
        assert info["kernel"] == capi.KERNEL_LDS_TILE and info["n_col_tiles"] == 1024
        assert (info["n_row_panels"] > 1) == (runs == 2), info
        dev = torch.device(DEV)
        W = d["W"].to(dev); H = d["H"].to(dev); out = torch.full((d["nnz"],), float("nan"), device=dev)
        plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
        torch.cuda.synchronize()
        outs[runs] = out.cpu()
    check(d, outs[1].numpy(), oracle, K)
    check(d, outs[2].numpy(), oracle, K)
    scale = float(np.abs(outs[1].numpy()).max())
    assert float((outs[1] - outs[2]).abs().max()) <= 1e-5 * scale
    # the same without short batches (the other stream layout), and through a plan file
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    o = capi.PlanOptions.defaults(ignore_env=1, kernel=capi.KERNEL_LDS_TILE, tile_size_x=16, tile_runs=2, tile_short_batches=0)
    plan = S.plan(K, options=o)
    assert plan.info()["n_row_panels"] > 1 and plan.info()["short_batches"] == 0
    dev = torch.device(DEV)
    W = d["W"].to(dev); H = d["H"].to(dev); out = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    check(d, out.cpu().numpy(), oracle, K)
    plan.save(tmp_path / "banded.plan")
    loaded = S.load_plan(tmp_path / "banded.plan", K, options=o)
    out2 = torch.full_like(out, float("nan"))
    loaded.execute(0, W.data_ptr(), H.data_ptr(), out2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("K,epilogue", [(256, "scale"), (512, "scale"), (384, "residual")])
def test_k_slices_inside_one_launch_or_one_launch_each(oracle, K, epilogue):
    """A sliced plan runs its K slices inside one kernel launch (fuse_slices = 1, what small matrices get) or one launch
    per slice; the arithmetic per position is the same, so the results agree bit for bit, in every value mode."""
    d = synth.make(3, 0.04, K=K, seed=11)
    dev = torch.device(DEV)
    W = d["W"].to(dev); H = d["H"].to(dev); dv = d["val"].to(dev)
    outs = {}
    for fuse in (0, 1):
        plan = host_plan(d, K, split_min_nnz=0, dense_blocks=0, fuse_slices=fuse)
        info = plan.info()
        assert info["k_slice"] == 128 and info["n_launches"] == (2 if fuse else 2 * K // 128), info
        res = []
        for val in (0, dv.data_ptr()):   # the plan's stream-order values / the caller's sorted values
            out = torch.full((d["nnz"],), float("nan"), device=dev)
            if epilogue == "scale":
                plan.execute(val, W.data_ptr(), H.data_ptr(), out.data_ptr())
            else:
                plan.execute_epilogue(val, W.data_ptr(), H.data_ptr(), out.data_ptr(), capi.EPILOGUE_RESIDUAL)
            torch.cuda.synchronize()
            res.append(out.cpu())
        assert torch.equal(res[0], res[1])
        outs[fuse] = res[0]
    assert torch.equal(outs[0], outs[1])
    if epilogue == "scale":
        check(d, outs[1].numpy(), oracle, K)
    else:
        residual_ok(outs[1].numpy(), d, oracle, K)


def test_concurrent_executes_on_one_plan_and_concurrent_plan_creation(oracle):
    """The header's promise: a plan is immutable, sddmm_execute may be called from several threads on the same plan
    (each on its own stream, outputs apart); plans may also be built concurrently."""
    import threading
    K = 128
    d = synth.make(3, 0.05, K=K, seed=19)
    dev = torch.device(DEV)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    opts = capi.PlanOptions.defaults(split_min_nnz=0, ignore_env=1)
    plan = S.plan(K, options=opts)
    W = d["W"].to(dev); H = d["H"].to(dev)
    ref = torch.empty(d["nnz"], device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), ref.data_ptr())
    torch.cuda.synchronize()
    check(d, ref.cpu().numpy(), oracle, K)
    n_threads, reps = 4, 8
    outs = [torch.full((d["nnz"],), float("nan"), device=dev) for _ in range(n_threads)]
    streams = [torch.cuda.Stream() for _ in range(n_threads)]
    errors = []

    def worker(i):
        try:
            for _ in range(reps):
                plan.execute(0, W.data_ptr(), H.data_ptr(), outs[i].data_ptr(), streams[i].cuda_stream)
            streams[i].synchronize()
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    th = [threading.Thread(target=worker, args=(i,)) for i in range(n_threads)]
    for t in th:
        t.start()
    for t in th:
        t.join()
    assert not errors, errors
    torch.cuda.synchronize()
    for o in outs:
        assert torch.equal(o, ref)
    # plans built at the same time from the same host matrix are the same plan
    plans = [None] * 3

    def builder(i):
        try:
            plans[i] = S.plan(K, options=opts)
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    th = [threading.Thread(target=builder, args=(i,)) for i in range(3)]
    for t in th:
        t.start()
    for t in th:
        t.join()
    assert not errors, errors
    for p in plans:
        o = torch.empty(d["nnz"], device=dev)
        p.execute(0, W.data_ptr(), H.data_ptr(), o.data_ptr())
        torch.cuda.synchronize()
        assert torch.equal(o, ref)


@pytest.mark.parametrize("K,softmax", [(256, False), (128, True), (256, True)])
def test_concurrent_executes_with_caller_workspaces(oracle, K, softmax):
    """sddmm_execute_ws takes the scratch memory (partial results between K slices, softmax records) from
    the caller: four threads run the same K-sliced plan at the same time, each with a workspace and a
    stream of its own, and every output has the bits of a lone call."""
    import threading
    d = synth.make(3, 0.05, K=K, seed=23)
    dev = torch.device(DEV)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    plan = S.plan(K, options=capi.PlanOptions.defaults(split_min_nnz=0, fuse_slices=0, ignore_env=1))
    assert plan.info()["k_slice"] == 128
    nbytes = plan.workspace_bytes()
    assert nbytes > 0 and nbytes % 256 == 0
    if K > 128:
        assert nbytes >= 4 * plan.info()["padded_positions"]
    W = d["W"].to(dev); H = d["H"].to(dev)
    form = capi.FORM_SOFTMAX if softmax else 0
    ref = torch.empty(d["nnz"], device=dev)
    if softmax:
        plan.execute_softmax(0, W.data_ptr(), H.data_ptr(), ref.data_ptr())
    else:
        plan.execute(0, W.data_ptr(), H.data_ptr(), ref.data_ptr())
    torch.cuda.synchronize()
    if not softmax:
        check(d, ref.cpu().numpy(), oracle, K)
    # too small a workspace, or none, is refused
    with pytest.raises(capi.SddmmError) as e:
        plan.execute_ws(0, W.data_ptr(), H.data_ptr(), ref.data_ptr(), 0, 0, form)
    assert e.value.code == capi.ERR_ARG
    n_threads, reps = 4, 6
    outs = [torch.full((d["nnz"],), float("nan"), device=dev) for _ in range(n_threads)]
    wss = [torch.full((nbytes // 4,), float("nan"), device=dev) for _ in range(n_threads)]
    streams = [torch.cuda.Stream() for _ in range(n_threads)]
    errors = []

    def worker(i):
        try:
            for _ in range(reps):
                plan.execute_ws(0, W.data_ptr(), H.data_ptr(), outs[i].data_ptr(), wss[i].data_ptr(), nbytes, form, streams[i].cuda_stream)
            streams[i].synchronize()
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    th = [threading.Thread(target=worker, args=(i,)) for i in range(n_threads)]
    for t in th:
        t.start()
    for t in th:
        t.join()
    assert not errors, errors
    torch.cuda.synchronize()
    for o in outs:
        assert torch.equal(o, ref)
    # the residual epilogue through the same entry point
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute_ws(0, W.data_ptr(), H.data_ptr(), out.data_ptr(), wss[0].data_ptr(), nbytes, capi.EPILOGUE_RESIDUAL)
    torch.cuda.synchronize()
    residual_ok(out.cpu().numpy(), d, oracle, K)


def test_workspace_entry_points_reject_bad_arguments():
    """sddmm_execute_ws and sddmm_plan_spmm check what they are given before anything is launched: a workspace that is
    missing, too small or not 256-byte aligned, unknown bits in `form`, the residual form without values, NULL arrays."""
    K = 256
    d = synth.make(3, 0.03, K=K, seed=13)
    dev = torch.device(DEV)
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev)
    opt = capi.PlanOptions.defaults(ignore_env=1, split_min_nnz=0, stage_factor=0, spmm_stream=1)
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), K, options=opt)  # no values
    nbytes = plan.workspace_bytes()
    assert nbytes > 0 and plan.info()["k_slice"] < K
    W = d["W"].to(dev); H = d["H"].to(dev); val = d["val"].to(dev)
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    ws = torch.empty(nbytes + 512, dtype=torch.uint8, device=dev)
    base = ws.data_ptr() + (-ws.data_ptr()) % 256
    args = (val.data_ptr(), W.data_ptr(), H.data_ptr(), out.data_ptr())

    def refused(call):
        with pytest.raises(capi.SddmmError) as e:
            call()
        assert e.value.code == capi.ERR_ARG, e.value
        torch.cuda.synchronize()
        assert bool(torch.isnan(out).all())  # nothing ran

    refused(lambda: plan.execute_ws(*args, 0, 0))                                   # no workspace
    refused(lambda: plan.execute_ws(*args, base, nbytes - 1))                       # too small
    refused(lambda: plan.execute_ws(*args, base + 16, nbytes))                      # misaligned
    refused(lambda: plan.execute_ws(*args, base, nbytes, 0x200))                    # unknown form bits
    refused(lambda: plan.execute_ws(*args, base, nbytes, 7))                        # unknown epilogue
    refused(lambda: plan.execute_ws(0, *args[1:], base, nbytes, capi.EPILOGUE_RESIDUAL))  # val - dot without values
    refused(lambda: plan.execute_ws(args[0], 0, args[2], args[3], base, nbytes))    # NULL W
    Y = torch.full((d["n_rows"], K), float("nan"), device=dev)
    x = torch.ones(d["nnz"], device=dev)
    for call in (lambda: plan.spmm(x.data_ptr(), H.data_ptr(), Y.data_ptr(), base, nbytes - 1),
                 lambda: plan.spmm(x.data_ptr(), H.data_ptr(), Y.data_ptr(), base + 16, nbytes),
                 lambda: plan.spmm(0, H.data_ptr(), Y.data_ptr()),
                 lambda: plan.spmm(x.data_ptr(), H.data_ptr(), 0)):
        with pytest.raises(capi.SddmmError) as e:
            call()
        assert e.value.code == capi.ERR_ARG, e.value
    torch.cuda.synchronize()
    assert bool(torch.isnan(Y).all())
    # and the good call still works afterwards
    plan.execute_ws(*args, base, nbytes)
    plan.spmm(x.data_ptr(), H.data_ptr(), Y.data_ptr(), base, nbytes)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(Y).all())
