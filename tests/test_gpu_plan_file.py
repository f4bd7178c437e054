"""Plan files (sddmm_plan_save / sddmm_plan_load / sddmm_plan_load_device): a loaded plan gives the
bits of the plan it was saved from, on the bag-of-words and the recommender shapes; a file is
refused for another matrix, K, option set or pattern; the command-line tool writes a plan beside
--save-bin and loads it on the next run."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

from sddmm_gpu_amd import capi, synth
from test_gpu_parity import check

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "sddmm_gpu_amd", "bin", "sddmm")


def run_plan(plan, d, dev, val=0):
    W = d["W"].to(dev); H = d["H"].to(dev)
    out = torch.full((d["nnz"],), float("nan"), device=dev)
    plan.execute(val, W.data_ptr(), H.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("cfg,scale,K,opts", [
    (2, 1.0, 256, {}), (3, 0.06, 128, {"split_min_nnz": 0}), (3, 0.03, 512, {"split_min_nnz": 0, "dense_blocks": 1, "dense_min_nnz": 1000}),
    (3, 0.03, 32, {"split_min_nnz": 0}), (1, 1.0, 32, {"kernel": capi.KERNEL_PANEL}), (1, 1.0, 32, {"kernel": capi.KERNEL_ROW_GATHER}),
    (2, 1.0, 100, {"kernel": capi.KERNEL_LDS_TILE, "tile_size_x": 64}),
])
def test_saved_plan_reproduces_the_fresh_plan(oracle, tmp_path, cfg, scale, K, opts):
    d = synth.make(cfg, scale, K=K)
    dev = torch.device("cuda:0")
    o = capi.PlanOptions.defaults(ignore_env=1, **opts)
    # (a) host-created plan: the file carries pattern and values
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    fresh = S.plan(K, options=o)
    ref = run_plan(fresh, d, dev)
    check(d, ref.cpu().numpy(), oracle, K)
    path = tmp_path / "host.plan"
    fresh.save(path)
    loaded = S.load_plan(path, K, options=o)
    li, fi = loaded.info(), fresh.info()
    for k in fi:
        if k not in ("plan_ms", "device_bytes"):
            assert li[k] == fi[k], k
    assert loaded.options() == fresh.options()
    assert torch.equal(run_plan(loaded, d, dev), ref)
    fresh.close()
    assert torch.equal(run_plan(loaded, d, dev), ref)   # nothing of the first plan is referenced
    # (b) device-created plan with values handed over: borrowed pattern, values inside the file
    rp = d["row_ptr"].to(dev); ci = d["col_ind"].to(dev); dv = d["val"].to(dev)
    p2 = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), K, options=o)
    ref_noval = run_plan(p2, d, dev)
    p2.set_values(dv.data_ptr())
    ref_val = run_plan(p2, d, dev)
    assert torch.equal(ref_val, ref)
    path2 = tmp_path / "dev.plan"
    p2.save(path2)
    p2.close()
    l2 = capi.Plan.load_device(path2, d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), K, options=o, keep=(rp, ci))
    assert torch.equal(run_plan(l2, d, dev), ref)
    assert torch.equal(run_plan(l2, d, dev, (dv * 2).data_ptr()), ref * 2)
    del ref_noval
    # a plan over a borrowed pattern cannot be loaded without it
    with pytest.raises(capi.SddmmError) as e:
        S.load_plan(path2, K, options=o)
    assert e.value.code == capi.ERR_ARG


def test_mismatched_key_is_rejected(tmp_path):
    d = synth.make(3, 0.03, K=64)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    o = capi.PlanOptions.defaults(ignore_env=1, tile_size_x=200)
    path = tmp_path / "a.plan"
    S.plan(64, options=o).save(path)
    assert S.load_plan(path, 64, options=o).info()["K"] == 64
    assert S.load_plan(path, 64, options=None).info()["K"] == 64           # None: any options
    for bad in (dict(K=128, options=o), dict(K=64, options=capi.PlanOptions.defaults(ignore_env=1, tile_size_x=100)),
                dict(K=64, options=capi.PlanOptions.defaults(ignore_env=1, tile_size_x=200, kernel=capi.KERNEL_ROW_GATHER))):
        with pytest.raises(capi.SddmmError) as e:
            S.load_plan(path, bad["K"], options=bad["options"])
        assert e.value.code == capi.ERR_FORMAT, bad
    # the same sizes, another pattern: one column index moved
    cols = d["col_ind"].numpy().copy()
    r0 = int(d["row_ptr"][1])  # last nonzero of the first non-empty row stays sorted when it moves to the last column
    rows = d["row_ind"].numpy()
    i = int(np.nonzero(np.diff(rows, append=rows[-1] + 1))[0][0])  # last position of the first row
    if cols[i] < d["n_cols"] - 1:
        cols[i] = d["n_cols"] - 1
    S2 = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], rows, cols, d["val"].numpy())
    assert S2.info()[3]
    with pytest.raises(capi.SddmmError) as e:
        S2.load_plan(path, 64, options=o)
    assert e.value.code == capi.ERR_FORMAT
    dev = torch.device("cuda:0")
    rp = d["row_ptr"].to(dev); ci = torch.from_numpy(cols).to(dev)
    p = capi.Plan.from_device_csr(d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), d["col_ind"].to(dev).data_ptr(), 64, options=o)
    path2 = tmp_path / "b.plan"
    p.save(path2)
    with pytest.raises(capi.SddmmError) as e:   # device hash of the changed pattern
        capi.Plan.load_device(path2, d["n_rows"], d["n_cols"], d["nnz"], rp.data_ptr(), ci.data_ptr(), 64, options=o)
    assert e.value.code == capi.ERR_FORMAT
    # not a plan file, a cut file, a missing file
    junk = tmp_path / "junk.plan"; junk.write_bytes(b"hello" * 100)
    cut = tmp_path / "cut.plan"; cut.write_bytes(path.read_bytes()[:5000])
    for f, code in ((junk, capi.ERR_FORMAT), (cut, capi.ERR_FORMAT), (tmp_path / "none.plan", capi.ERR_IO)):
        with pytest.raises(capi.SddmmError) as e:
            S.load_plan(f, 64, options=o)
        assert e.value.code == code


def test_damaged_and_foreign_files_are_rejected(tmp_path):
    """One flipped byte anywhere in the launch table or in the arrays, or the build id of another
    library build, and the file is refused before anything is launched; nothing is left under the
    plan's name by a save that could not finish."""
    d = synth.make(3, 0.03, K=128)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    o = capi.PlanOptions.defaults(ignore_env=1, split_min_nnz=0)
    path = tmp_path / "good.plan"
    S.plan(128, options=o).save(path)
    assert not os.path.exists(str(path) + ".tmp")
    good = path.read_bytes()
    assert S.load_plan(path, 128, options=o).info()["K"] == 128
    n = len(good)
    build_at = good.index(b"sddmm-")  # the build id inside the header
    spots = {"launch table": 600, "arrays, early": n // 3, "arrays, late": n - 5, "checksum": build_at + 40 + 9,
             "build id": build_at + 8}
    for what, at in spots.items():
        bad = bytearray(good)
        bad[at] ^= 0x10
        f = tmp_path / "bad.plan"
        f.write_bytes(bytes(bad))
        with pytest.raises(capi.SddmmError) as e:
            S.load_plan(f, 128, options=o)
        assert e.value.code == capi.ERR_FORMAT, what
    # a save into a directory that does not exist fails cleanly
    with pytest.raises(capi.SddmmError) as e:
        S.plan(128, options=o).save(tmp_path / "no_such_dir" / "x.plan")
    assert e.value.code == capi.ERR_IO


def test_cli_saves_and_reloads_the_plan(oracle, tmp_path):
    d = synth.make(2, 0.5)
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    mtx = tmp_path / "bow.mtx"; S.write_mtx(mtx)
    K = 64
    cpu = oracle.sddmm_csr(d["row_ptr"].numpy(), d["col_ind"].numpy(), d["val"].numpy(), oracle.initial(d["n_rows"], K),
                           oracle.initial(d["n_cols"], K))
    vec = tmp_path / "o.f32"; cpu.tofile(vec)
    binf = tmp_path / "bow.bin"
    r = subprocess.run([CLI, str(mtx), str(K), "192", "0", "--save-bin", str(binf), "--json", "--check-against", str(vec)],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr + r.stdout
    assert os.path.exists(str(binf) + f".k{K}.x192.y0.0.plan")
    js = json.loads([ln for ln in r.stdout.splitlines() if ln.startswith("{")][0])
    assert js["plan_loaded"] is False and js["mismatches"] == 0
    r = subprocess.run([CLI, str(binf), str(K), "192", "0", "--json", "--check-against", str(vec)], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stderr + r.stdout
    js2 = json.loads([ln for ln in r.stdout.splitlines() if ln.startswith("{")][0])
    assert js2["plan_loaded"] is True and js2["mismatches"] == 0 and "plan loaded from" in r.stderr
    assert js2["tile_size_x"] == js["tile_size_x"] and js2["checksum"] == js["checksum"]
    # other arguments: no such plan file, a fresh plan is built
    r = subprocess.run([CLI, str(binf), str(K), "100", "0", "--json", "--check-against", str(vec)], capture_output=True, text=True,
                       timeout=120)
    js3 = json.loads([ln for ln in r.stdout.splitlines() if ln.startswith("{")][0])
    assert r.returncode == 0 and js3["plan_loaded"] is False and js3["mismatches"] == 0
