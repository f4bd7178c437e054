"""The forms around the SDDMM on the GPU, through the C ABI: row-wise softmax of the sampled
products (on its own and as sddmm_execute_softmax) and the CSR SpMM that consumes them, against the
CPU oracle.  Softmax: relative 1e-5 per entry (terms are positive: no cancellation).  SpMM:
1e-5*sqrt(row length) relative to sum|x*h| (signed terms)."""
import numpy as np
import pytest
import torch

from sddmm_gpu_amd import capi, synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def softmax_ok(got, want):
    assert got.shape == want.shape and np.all(np.isfinite(got))
    bad = np.abs(got.astype(np.float64) - want) > 1e-5 * np.abs(want) + 1e-37
    assert not bad.any(), (int(bad.sum()), float(np.abs(got - want).max()))


@pytest.mark.parametrize("cfg,scale", [(1, 1.0), (2, 1.0), (3, 0.05), (5, 2.0 ** -6)])
def test_row_softmax_matches_oracle(oracle, cfg, scale):
    d = synth.make(cfg, scale)
    dev = torch.device(DEV)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(d["nnz"], generator=g) * 4.0
    rp = d["row_ptr"].to(dev); xd = x.to(dev); out = torch.full_like(xd, float("nan"))
    capi.row_softmax(d["n_rows"], rp.data_ptr(), xd.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    want = oracle.row_softmax(d["row_ptr"].numpy(), x.numpy())
    softmax_ok(out.cpu().numpy(), want)
    # in place, and the closed form: equal logits -> 1 / row length
    capi.row_softmax(d["n_rows"], rp.data_ptr(), xd.data_ptr(), xd.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(xd, out)
    ones = torch.full((d["nnz"],), 3.25, device=dev)
    capi.row_softmax(d["n_rows"], rp.data_ptr(), ones.data_ptr(), ones.data_ptr())
    deg = np.diff(d["row_ptr"].numpy())
    assert np.allclose(ones.cpu().numpy(), 1.0 / deg[d["row_ind"].numpy()], rtol=1e-6, atol=0)


@pytest.mark.parametrize("misalign", [0, 1])
def test_row_softmax_edge_rows(oracle, misalign):
    """Rows at the boundaries of the kernel's cases: rows of up to 4096 entries are grouped into chunks of whole rows, a wave
    takes a chunk 64 rows at a time and gives a row to a lane (up to 8 entries), 8 lanes (up to 96), 32 lanes (up to 512)
    or all its lanes (up to 1024 in registers, beyond that in two walks); longer rows go to workgroups of their own (next
    test).  The runs of empty rows span several chunks' worth of row pointers."""
    lens = ([0, 1, 0, 8, 9, 64, 65, 96, 97, 192, 193, 512, 513, 1023, 1024, 1025, 0, 2, 511]      # every class, whole rows
            + [2 * 4096 - sum([1, 8, 9, 64, 65, 96, 97, 192, 193, 512, 513, 1023, 1024, 1025, 2, 511])]  # ... up to the end of chunk 1 exactly
            + [4096]                                                        # a row that is exactly chunk 2
            + [5000, 3]                                                     # a row over two chunk boundaries, then a short one
            + [0] * 6000 + [1, 2] * 700 + [0] * 5000                        # runs of empty rows longer than a staging round
            + [13000]                                                       # a row over three boundaries with whole chunks inside
            + [2] * 3000 + [7, 0, 300, 5])
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    rng = np.random.default_rng(1)
    x = rng.normal(0, 10, rp[-1]).astype(np.float32)
    x[rp[5]] = 80.0; x[rp[lens.index(5000)] + 17] = -90.0; x[rp[lens.index(13000)] + 12000] = 75.0
    dev = torch.device(DEV)
    # (misalign: x and out start 4 bytes past a 16-byte boundary, which takes the kernels' scalar load/store path)
    xbuf = torch.zeros(len(x) + 4, device=dev); obuf = torch.full((len(x) + 4,), float("nan"), device=dev)
    xd = xbuf[misalign:misalign + len(x)]; out = obuf[misalign:misalign + len(x)]
    xd.copy_(torch.from_numpy(x))
    capi.row_softmax(len(lens), torch.from_numpy(rp).to(dev).data_ptr(), xd.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    softmax_ok(out.cpu().numpy(), oracle.row_softmax(rp, x))
    assert bool(torch.isnan(obuf[:misalign]).all()) and bool(torch.isnan(obuf[misalign + len(x):]).all())  # nothing written outside
    capi.row_softmax(0, 0, 0, 0)  # nothing to do
    empty_rp = torch.zeros(6, dtype=torch.int32, device=dev)  # five rows, no entries
    capi.row_softmax(5, empty_rp.data_ptr(), xd.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    assert bool(torch.isnan(obuf[:misalign]).all())  # (and nothing was written)


@pytest.mark.parametrize("misalign", [0, 1, 2])
def test_row_softmax_long_rows(oracle, misalign):
    """Rows of more than a chunk (4096 entries) and up to 65,528 are held in registers by one workgroup each (up to
    16,376 entries with 4 float4 per thread, beyond that with 16); longer ones go through the chunk records.  The cases:
    the limits on both sides, a long row that starts exactly on a chunk boundary, long rows back to back, short rows
    squeezed between them, a long row that ends the array (its last float4 is cut by the end of x)."""
    lens = ([5, 4097, 3, 4096, 4098]                 # just over a chunk; a whole-chunk row is not long
            + [4096 * 6 - (5 + 4097 + 3 + 4096 + 4098)]  # fill up to a chunk boundary ...
            + [5000]                                 # ... so that this long row starts exactly on it
            + [16376, 16377, 1, 0, 2]                # the two register classes
            + [65528, 9000, 65529, 7]                # the longest long row, one after it, the shortest cut row
            + [300] * 40 + [12345])                  # ordinary rows, and a long row at the end of the array
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    assert rp[-1] % 4 != 0  # (the array ends inside a float4)
    rng = np.random.default_rng(2)
    x = rng.normal(0, 6, rp[-1]).astype(np.float32)
    x[rp[lens.index(65528)] + 60000] = 70.0; x[rp[lens.index(65529)] + 3] = 66.0; x[rp[-1] - 1] = 50.0
    dev = torch.device(DEV)
    xbuf = torch.zeros(len(x) + 8, device=dev); obuf = torch.full((len(x) + 8,), float("nan"), device=dev)
    xd = xbuf[misalign:misalign + len(x)]; out = obuf[misalign:misalign + len(x)]
    xd.copy_(torch.from_numpy(x))
    rpd = torch.from_numpy(rp).to(dev)
    capi.row_softmax(len(lens), rpd.data_ptr(), xd.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    want = oracle.row_softmax(rp, x)
    softmax_ok(out.cpu().numpy(), want)
    assert bool(torch.isnan(obuf[:misalign]).all()) and bool(torch.isnan(obuf[misalign + len(x):]).all())  # nothing written outside
    # in place; and input aligned with output not (and the other way round)
    capi.row_softmax(len(lens), rpd.data_ptr(), xd.data_ptr(), xd.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(xd, out)
    xd.copy_(torch.from_numpy(x))
    other = torch.full((len(x) + 8,), float("nan"), device=dev)
    o2 = other[3 - misalign:3 - misalign + len(x)]
    capi.row_softmax(len(lens), rpd.data_ptr(), xd.data_ptr(), o2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(o2, out)
    assert bool(torch.isnan(other[:3 - misalign]).all()) and bool(torch.isnan(other[3 - misalign + len(x):]).all())


def test_row_softmax_mostly_empty_rows(oracle):
    """A chunk of 4096 entries that spans far more rows than the average chunk (mostly empty rows) is not left to its own
    wave: that wave takes twice the average number of rows (at least 2048), the rest is dealt out to all workgroups in
    parts of 512 rows.  Here: ordinary rows, then 2.6 million rows with one to three entries in every 997th (more parts
    than there are workgroups, so some take two), then ordinary rows again, a second such stretch with rows of every
    short class in it, and the array ends inside a stretch of empty rows."""
    rng = np.random.default_rng(5)
    sparse = np.zeros(2_600_000, dtype=np.int64); sparse[::997] = rng.integers(1, 4, len(sparse[::997]))
    second = np.zeros(400_000, dtype=np.int64); second[::15011] = np.resize([1, 8, 9, 96, 97, 512, 513, 1100], len(second[::15011]))
    lens = np.concatenate([rng.integers(50, 150, 3000), sparse, rng.integers(0, 300, 2000), second, [7], np.zeros(70_000, dtype=np.int64)])
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    x = rng.normal(0, 5, rp[-1]).astype(np.float32)
    dev = torch.device(DEV)
    xd = torch.from_numpy(x).to(dev); out = torch.full_like(xd, float("nan")); rpd = torch.from_numpy(rp).to(dev)
    for _ in range(2):  # (the second call finds the first one's list in the library's arrays)
        out.fill_(float("nan"))
        capi.row_softmax(len(lens), rpd.data_ptr(), xd.data_ptr(), out.data_ptr())
        torch.cuda.synchronize()
        softmax_ok(out.cpu().numpy(), oracle.row_softmax(rp, x))


@pytest.mark.parametrize("kind", ["heavy tail", "huge rows among empty ones", "chunks with both", "class limits"])
def test_row_softmax_mixed_lengths(oracle, kind):
    """Row-length mixes that put several of the pass's cases into the same chunks: a heavy-tailed distribution; rows of
    tens of thousands of entries between long runs of empty rows; stretches of mostly empty rows that a huge row runs
    into (the chunk is then in the last kernel's list for both reasons); rows at the limits of every class."""
    rng = np.random.default_rng(11)
    if kind == "heavy tail":
        lens = np.minimum((rng.pareto(0.8, 40_000) * 3).astype(np.int64), 300_000)
    elif kind == "huge rows among empty ones":
        lens = np.zeros(600_000, dtype=np.int64)
        at = rng.choice(len(lens), 200, replace=False)
        lens[at] = rng.choice([1, 5, 100, 3000, 5000, 17_000, 40_000], 200)
    elif kind == "chunks with both":
        lens = np.zeros(1_500_000, dtype=np.int64)
        lens[::len(lens) // 37] = 50_000
        lens[5::997] = 3
    else:
        lens = rng.choice([4095, 4096, 4097, 8191, 8192, 8193, 16_376, 16_377, 12_288, 1, 0], 300)
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    x = rng.normal(0, 6, rp[-1]).astype(np.float32)
    dev = torch.device(DEV)
    xd = torch.from_numpy(x).to(dev); out = torch.full_like(xd, float("nan")); rpd = torch.from_numpy(rp).to(dev)
    capi.row_softmax(len(lens), rpd.data_ptr(), xd.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    softmax_ok(out.cpu().numpy(), oracle.row_softmax(rp, x))


@pytest.mark.parametrize("kernel,K", [("auto", 128), ("auto", 64), ("row", 100), ("lds", 32), ("panel", 64)])
def test_execute_softmax_matches_oracle(oracle, kernel, K):
    kid = {"auto": capi.KERNEL_AUTO, "row": capi.KERNEL_ROW_GATHER, "lds": capi.KERNEL_LDS_TILE, "panel": capi.KERNEL_PANEL}[kernel]
    d = synth.make(3, 0.03, K=K, seed=12)
    d["W"] = d["W"] * 8.0; d["H"] = d["H"] * 8.0  # logits of order one
    dev = torch.device(DEV)
    W = d["W"].to(dev); H = d["H"].to(dev)
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    cpu_logits = oracle.sddmm_csr(d["row_ptr"].numpy(), d["col_ind"].numpy(), d["val"].numpy(), d["W"].numpy(), d["H"].numpy())
    want = oracle.row_softmax(d["row_ptr"].numpy(), cpu_logits)
    # host-created plan (values inside) and device-created plan (values at execute)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    opt = capi.PlanOptions.defaults(ignore_env=1, kernel=kid, split_min_nnz=0)
    plan = S.plan(K, options=opt)
    plan.execute_softmax(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    # the logits differ from the oracle's by the SDDMM tolerance; a softmax entry moves by at most that (absolute, in the logit)
    tol = 1e-5 * np.sqrt(K) * np.abs(cpu_logits).max() * 4 + 1e-5
    assert np.all(np.isfinite(got)) and np.all(np.abs(got - want) <= tol * want + 1e-37)
    sums = np.bincount(d["row_ind"].numpy(), weights=got.astype(np.float64), minlength=d["n_rows"])
    assert np.allclose(sums[np.diff(d["row_ptr"].numpy()) > 0], 1.0, atol=1e-5)
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev); dv = d["val"].to(dev)
    p2 = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), K, options=opt)
    out2 = torch.full_like(out, float("nan"))
    p2.execute_softmax(dv.data_ptr(), W.data_ptr(), H.data_ptr(), out2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    # the two-call form gives the same bits
    plan.execute(0, W.data_ptr(), H.data_ptr(), out2.data_ptr())
    capi.row_softmax(d["n_rows"], rp.data_ptr(), out2.data_ptr(), out2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("cfg,scale,K", [(1, 1.0, 32), (2, 1.0, 256), (3, 0.05, 128), (3, 0.02, 100), (3, 0.02, 7), (3, 0.02, 36),
                                         (5, 2.0 ** -6, 512), (3, 0.01, 2048), (3, 0.01, 2052)])
def test_spmm_matches_oracle(oracle, cfg, scale, K):
    d = synth.make(cfg, scale, K=K)
    dev = torch.device(DEV)
    g = torch.Generator().manual_seed(K)
    x = torch.randn(d["nnz"], generator=g)
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev); xd = x.to(dev); H = d["H"].to(dev).contiguous()
    Y = torch.full((d["n_rows"], K), float("nan"), device=dev)
    capi.spmm_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), xd.data_ptr(), K, H.data_ptr(), Y.data_ptr())
    torch.cuda.synchronize()
    want, absy = oracle.spmm_csr(d["row_ptr"].numpy(), d["col_ind"].numpy(), x.numpy(), d["H"].numpy(), with_abs=True)
    got = Y.cpu().numpy()
    assert np.all(np.isfinite(got))
    deg = np.diff(d["row_ptr"].numpy()).astype(np.float64)
    bound = 1e-5 * np.sqrt(np.maximum(deg, 1.0))[:, None] * absy + 1e-30
    bad = np.abs(got.astype(np.float64) - want) > bound
    assert not bad.any(), (int(bad.sum()), float(np.abs(got - want).max()))
    assert np.all(got[deg == 0] == 0)
    # closed form: H of ones -> every output column is the row sum of x
    ones = torch.ones_like(H)
    capi.spmm_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), xd.data_ptr(), K, ones.data_ptr(), Y.data_ptr())
    torch.cuda.synchronize()
    rs = np.bincount(d["row_ind"].numpy(), weights=x.numpy().astype(np.float64), minlength=d["n_rows"])
    ab = np.bincount(d["row_ind"].numpy(), weights=np.abs(x.numpy()).astype(np.float64), minlength=d["n_rows"])
    assert np.all(np.abs(Y.cpu().numpy()[:, K // 2] - rs) <= 1e-5 * np.sqrt(np.maximum(deg, 1.0)) * ab + 1e-30)


def test_attention_chain_and_errors(oracle):
    """softmax(S .* W H^T) H end to end on the bag-of-words shape, and the argument checks."""
    K = 64
    d = synth.make(2, 0.5, K=K)
    d["W"] = d["W"] * 3.0
    dev = torch.device(DEV)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), np.ones(d["nnz"], np.float32))
    plan = S.plan(K)
    W = d["W"].to(dev); H = d["H"].to(dev); rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev)
    att = torch.empty(d["nnz"], device=dev); Y = torch.empty(d["n_rows"], K, device=dev)
    plan.execute_softmax(0, W.data_ptr(), H.data_ptr(), att.data_ptr())
    capi.spmm_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), att.data_ptr(), K, H.data_ptr(), Y.data_ptr())
    torch.cuda.synchronize()
    logits = oracle.sddmm_csr(d["row_ptr"].numpy(), d["col_ind"].numpy(), np.ones(d["nnz"], np.float32), d["W"].numpy(), d["H"].numpy())
    want = oracle.spmm_csr(d["row_ptr"].numpy(), d["col_ind"].numpy(), oracle.row_softmax(d["row_ptr"].numpy(), logits), d["H"].numpy())
    # a convex combination of H rows: compare against the scale of H
    assert np.abs(Y.cpu().numpy() - want).max() <= 1e-4 * np.abs(d["H"].numpy()).max()
    with pytest.raises(capi.SddmmError) as e:
        capi.spmm_csr(5, 5, 3, rp.data_ptr(), 0, 0, K, 0, Y.data_ptr())
    assert e.value.code == capi.ERR_ARG
    with pytest.raises(capi.SddmmError) as e:
        capi.spmm_csr(5, 5, 3, rp.data_ptr(), ci.data_ptr(), att.data_ptr(), 0, H.data_ptr(), Y.data_ptr())
    assert e.value.code == capi.ERR_ARG
    with pytest.raises(capi.SddmmError) as e:
        capi.row_softmax(5, 0, att.data_ptr(), att.data_ptr())
    assert e.value.code == capi.ERR_ARG


def spmm_ok(oracle, d, x, got, K):
    want, absy = oracle.spmm_csr(d["row_ptr"].numpy(), d["col_ind"].numpy(), x.numpy(), d["H"].numpy(), with_abs=True)
    assert np.all(np.isfinite(got))
    deg = np.diff(d["row_ptr"].numpy()).astype(np.float64)
    bound = 1e-5 * np.sqrt(np.maximum(deg, 1.0))[:, None] * absy + 1e-30
    bad = np.abs(got.astype(np.float64) - want) > bound
    assert not bad.any(), (int(bad.sum()), float(np.abs(got - want).max()))
    assert np.all(got[deg == 0] == 0)


@pytest.mark.parametrize("cfg,scale,K,opts", [
    (3, 0.05, 128, {"split_min_nnz": 0}), (3, 0.05, 128, {"split_min_nnz": 0, "tile_few_blocks": 0}),
    (3, 0.03, 256, {"split_min_nnz": 0}), (3, 0.03, 64, {"split_min_nnz": 0, "stage_factor": 0}), (3, 0.03, 32, {"split_min_nnz": 0, "stage_factor": 0}),
    (2, 1.0, 256, {}), (2, 1.0, 128, {"tile_size_x": 192}), (5, 2.0 ** -6, 128, {}), (5, 2.0 ** -6, 512, {"tile_runs": 1}),
    (1, 1.0, 32, {"kernel": capi.KERNEL_LDS_TILE})])
def test_plan_spmm_on_the_tile_stream(oracle, cfg, scale, K, opts):
    """Y = X H on the plan's column tiles (spmm_stream = 1): against the oracle, the same bits on
    every call and with a caller's workspace, and the SDDMM of the same plan unchanged."""
    d = synth.make(cfg, scale, K=K)
    dev = torch.device(DEV)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    plan = S.plan(K, options=capi.PlanOptions.defaults(ignore_env=1, spmm_stream=1, **opts))
    info = plan.info()
    assert info["spmm_runs"] > 0, info
    g = torch.Generator().manual_seed(K + cfg)
    x = torch.randn(d["nnz"], generator=g)
    xd = x.to(dev); H = d["H"].to(dev).contiguous(); W = d["W"].to(dev)
    Y = torch.full((d["n_rows"], K), float("nan"), device=dev)
    plan.spmm(xd.data_ptr(), H.data_ptr(), Y.data_ptr())
    torch.cuda.synchronize()
    spmm_ok(oracle, d, x, Y.cpu().numpy(), K)
    Y2 = torch.full((d["n_rows"], K), float("nan"), device=dev)
    plan.spmm(xd.data_ptr(), H.data_ptr(), Y2.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(Y, Y2)
    nbytes = plan.workspace_bytes()
    assert nbytes >= 4 * K // max(1, K // info["k_slice"]) * info["spmm_runs"]
    ws = torch.full((nbytes // 4,), float("nan"), device=dev)
    Y3 = torch.full((d["n_rows"], K), float("nan"), device=dev)
    plan.spmm(xd.data_ptr(), H.data_ptr(), Y3.data_ptr(), ws.data_ptr(), nbytes)
    torch.cuda.synchronize()
    assert torch.equal(Y, Y3)
    # closed form: H of ones -> every output column is the row sum of x
    ones = torch.ones_like(H)
    plan.spmm(xd.data_ptr(), ones.data_ptr(), Y.data_ptr())
    torch.cuda.synchronize()
    deg = np.diff(d["row_ptr"].numpy()).astype(np.float64)
    rs = np.bincount(d["row_ind"].numpy(), weights=x.numpy().astype(np.float64), minlength=d["n_rows"])
    ab = np.bincount(d["row_ind"].numpy(), weights=np.abs(x.numpy()).astype(np.float64), minlength=d["n_rows"])
    assert np.all(np.abs(Y.cpu().numpy()[:, K - 1] - rs) <= 1e-5 * np.sqrt(np.maximum(deg, 1.0)) * ab + 1e-30)
    # the plan's SDDMM is what it was
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(0, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    from test_gpu_parity import check
    check(d, out.cpu().numpy(), oracle, K)


def test_plan_spmm_without_a_tile_stream_takes_the_csr_path(oracle):
    K = 64
    d = synth.make(3, 0.02, K=K)
    dev = torch.device(DEV)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    x = torch.randn(d["nnz"], generator=torch.Generator().manual_seed(3))
    xd = x.to(dev); H = d["H"].to(dev).contiguous()
    for opts in ({}, {"kernel": capi.KERNEL_ROW_GATHER, "spmm_stream": 1}):
        plan = S.plan(K, options=capi.PlanOptions.defaults(ignore_env=1, **opts))
        assert plan.info()["spmm_runs"] == 0
        Y = torch.full((d["n_rows"], K), float("nan"), device=dev)
        plan.spmm(xd.data_ptr(), H.data_ptr(), Y.data_ptr())
        torch.cuda.synchronize()
        spmm_ok(oracle, d, x, Y.cpu().numpy(), K)
