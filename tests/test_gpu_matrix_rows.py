"""The matrix-core share of a tile launch: the heaviest rows leave the stream and are computed as
32 x 32 blocks (fp32 MFMA) by extra waves of the tile kernel's own workgroups.  Parity with the
CPU oracle in every value mode and epilogue, for each split of the workgroup between vector and
matrix-core waves, and the bookkeeping of the plan."""
import numpy as np
import pytest
import torch

from conftest import parity_report
from sddmm_gpu_amd import capi, synth
from test_gpu_parity import check, residual_ok

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def forced(**kw):
    # a scaled recommender shape is small: force the two-class split, the die-local assignment
    # and the matrix-core share that the planner chooses by itself at full size
    return capi.PlanOptions.defaults(ignore_env=1, split_min_nnz=0, stage_factor=0, tile_few_blocks=0, matrix_rows=1, **kw)


@pytest.mark.parametrize("waves", [(12, 4), (8, 8), (8, 4)])
@pytest.mark.parametrize("scale,permille", [(0.1, 100), (0.06, 60)])
def test_matrix_rows_every_value_mode(oracle, waves, scale, permille):
    K = 128
    d = synth.make(3, scale, K=K, seed=11)
    dev = torch.device(DEV)
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev)
    opts = forced(matrix_permille=permille, tile_waves=waves[0], matrix_waves=waves[1])
    plan = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), K, keep=(rp, ci),
                                     options=opts)
    info = plan.info()
    assert info["matrix_rows"] >= 256 and info["matrix_rows"] % 256 == 0, info
    assert info["matrix_nnz"] > d["nnz"] // 20, info
    assert info["block"] == 64 * sum(waves), info
    assert info["dense_nnz"] + sum(info["class_nnz"]) == d["nnz"]
    W = d["W"].to(dev); H = d["H"].to(dev); dv = d["val"].to(dev)
    rows = d["row_ind"].numpy(); cols = d["col_ind"].numpy(); vals = d["val"].numpy()
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    # no values at all
    plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    cpu1 = oracle.sddmm_coo(rows, cols, vals, d["W"].numpy(), d["H"].numpy(), apply_val=False)
    _, absp1 = oracle.sddmm_f64(rows, cols, np.ones_like(vals), d["W"].numpy(), d["H"].numpy())
    assert np.all(np.isfinite(out.cpu().numpy()))
    assert parity_report(out.cpu().numpy(), cpu1, K, absp1)["violations"] == 0
    # values passed at execute (sorted order)
    out.fill_(float("nan"))
    plan.execute(dv.data_ptr(), W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    check(d, out.cpu().numpy(), oracle, K)
    # values owned by the plan (stream order for the vector waves, sorted order for the matrix-core waves)
    plan.set_values(dv.data_ptr())
    out2 = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), out2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    # a second call gives the same bits (no atomics, no order dependence)
    out3 = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), out3.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(out2, out3)
    # the packed operands in a caller's workspace instead of the plan's
    nbytes = plan.workspace_bytes()
    assert nbytes >= 16384 * (info["matrix_rows"] // 32 + (d["n_cols"] + 31) // 32)
    ws = torch.full((nbytes // 4,), float("nan"), device=dev)
    out4 = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute_ws(0, W.data_ptr(), H.data_ptr(), out4.data_ptr(), ws.data_ptr(), nbytes)
    torch.cuda.synchronize()
    assert torch.equal(out4, out2)
    for src in (0, dv.data_ptr()):
        out.fill_(float("nan"))
        plan.execute_epilogue(src, W.data_ptr(), H.data_ptr(), out.data_ptr(), capi.EPILOGUE_RESIDUAL)
        torch.cuda.synchronize()
        residual_ok(out.cpu().numpy(), d, oracle, K)


def test_matrix_rows_off_and_host_plan(oracle):
    """matrix_rows = 0 keeps every row in the stream; a plan made from a host matrix carries its
    values to both kinds of waves."""
    K = 128
    d = synth.make(3, 0.1, K=K, seed=12)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    off = S.plan(K, options=capi.PlanOptions.defaults(ignore_env=1, split_min_nnz=0, tile_few_blocks=0, matrix_rows=0))
    assert off.info()["matrix_nnz"] == 0 and off.info()["matrix_rows"] == 0
    on = S.plan(K, options=forced(matrix_permille=100))
    assert on.info()["matrix_nnz"] > 0
    assert on.info()["padded_positions"] < off.info()["padded_positions"]
    dev = torch.device(DEV)
    W = d["W"].to(dev); H = d["H"].to(dev)
    for plan in (off, on):
        out = torch.full((d["nnz"],), float("nan"), device=dev)
        plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
        torch.cuda.synchronize()
        check(d, out.cpu().numpy(), oracle, K)


def test_matrix_rows_edge_columns(oracle):
    """n_cols not a multiple of 32 (the last column block is part empty), rows that are completely
    full, and columns nobody uses."""
    K = 128
    rng = np.random.default_rng(5)
    n_rows, n_cols = 3000, 1000 + 13
    dens = np.concatenate([np.full(40, 1.0), rng.uniform(0.3, 0.95, 400), rng.uniform(0.0, 0.05, n_rows - 440)])
    rng.shuffle(dens)
    mask = rng.random((n_rows, n_cols)) < dens[:, None]
    mask[:, 500:520] = False  # unused columns
    mask[dens == 1.0, :] = True
    mask[dens == 1.0, 500:520] = False
    r, c = np.nonzero(mask)
    d = dict(n_rows=n_rows, n_cols=n_cols, nnz=len(r), K=K, row_ind=torch.from_numpy(r.astype(np.int32)),
             col_ind=torch.from_numpy(c.astype(np.int32)),
             row_ptr=torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(r, minlength=n_rows))]).astype(np.int32)),
             val=torch.from_numpy(rng.standard_normal(len(r)).astype(np.float32)),
             W=torch.from_numpy(rng.standard_normal((n_rows, K)).astype(np.float32)),
             H=torch.from_numpy(rng.standard_normal((n_cols, K)).astype(np.float32)))
    S = capi.Coo.from_arrays(n_rows, n_cols, r.astype(np.int32), c.astype(np.int32), d["val"].numpy())
    plan = S.plan(K, options=forced(matrix_permille=250, short_row_max=1))
    info = plan.info()
    assert info["matrix_rows"] == 256, info
    dev = torch.device(DEV)
    W = d["W"].to(dev); H = d["H"].to(dev)
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    check(d, out.cpu().numpy(), oracle, K)
