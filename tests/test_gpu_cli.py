"""The sddmm command-line driver on the GPU: the reference's calling
convention (sddmm input K tile_size_X tile_size_Y), its three output lines,
and the result checked through the --json checksum against the CPU oracle run
with the reference's own dense factors (0.1*drand48())."""
import json
import os
import re
import subprocess

import numpy as np
import pytest

from sddmm_gpu_amd import capi, synth

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "sddmm_gpu_amd", "bin", "sddmm")


def test_cli_matches_oracle(oracle, tmp_path):
    assert os.path.exists(CLI), "build the CLI with make -C sddmm_gpu_amd/csrc"
    d = synth.make(2, 0.5)
    rows = d["row_ind"].numpy(); cols = d["col_ind"].numpy(); vals = d["val"].numpy()
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], rows, cols, vals)
    mtx = tmp_path / "bow.mtx"
    S.write_mtx(mtx)
    K = 64
    W = oracle.initial(d["n_rows"], K); H = oracle.initial(d["n_cols"], K)
    expect = oracle.sddmm_csr(d["row_ptr"].numpy(), cols, vals, W, H).astype(np.float64).sum()
    for extra, tx, ty in (([], 192, 50000), (["--kernel", "row"], 0, 0), (["--kernel", "lds"], 64, 32)):
        r = subprocess.run([CLI, str(mtx), str(K), str(tx), str(ty), "--json", "--runs", "3"] + extra, capture_output=True,
                           text=True, timeout=120)
        assert r.returncode == 0, r.stderr
        out = r.stdout
        m = re.search(r"Matrix info:\s+rows: (\d+), cols: (\d+), nnz: (\d+)", out)
        assert m and tuple(map(int, m.groups())) == (d["n_rows"], d["n_cols"], d["nnz"])
        assert re.search(r"Tilesize: X = \d+, tilesize: Y = \d+, TB: \d+", out)
        m = re.search(r"Time for SDDMM with K = (\d+) : ([0-9.eE+-]+) ms", out)
        assert m and int(m.group(1)) == K and float(m.group(2)) > 0
        js = json.loads([ln for ln in out.splitlines() if ln.startswith("{")][0])
        assert js["nnz"] == d["nnz"] and js["K"] == K
        assert abs(js["checksum"] - expect) <= 1e-5 * np.sqrt(K) * abs(expect) + 1e-6, (js["checksum"], expect)


def test_cli_column_sorted_input_and_errors(oracle, tmp_path):
    rng = np.random.default_rng(5)
    n, m = 60, 90
    keys = np.unique(rng.integers(0, n * m, 700))
    rows, cols = (keys // m).astype(np.int32), (keys % m).astype(np.int32)
    order = np.lexsort((rows, cols))  # column-sorted file, as the reference's conversion expects
    vals = rng.random(len(keys)).astype(np.float32) + 0.5
    p = tmp_path / "colsorted.mtx"
    capi.Coo.from_arrays(n, m, rows[order], cols[order], vals[order]).write_mtx(p)
    r = subprocess.run([CLI, str(p), "32", "16", "8", "--transpose", "--json"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert f"rows: {m}, cols: {n}, nnz: {len(keys)}" in r.stdout
    t_r, t_c, t_v, rp = oracle.transpose_sort(rows[order], cols[order], vals[order], m)
    W = oracle.initial(m, 32); H = oracle.initial(n, 32)
    expect = oracle.sddmm_csr(rp, t_c, t_v, W, H).astype(np.float64).sum()
    js = json.loads([ln for ln in r.stdout.splitlines() if ln.startswith("{")][0])
    assert abs(js["checksum"] - expect) <= 1e-4 * abs(expect)
    # errors: missing file, bad K
    r = subprocess.run([CLI, str(tmp_path / "nope.mtx"), "32", "0", "0"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "cannot open" in r.stderr
    r = subprocess.run([CLI, str(p), "0", "0", "0"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0
    r = subprocess.run([CLI], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "usage" in r.stderr
