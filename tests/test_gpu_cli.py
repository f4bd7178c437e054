"""The sddmm command-line driver on the GPU: the reference's calling
convention (sddmm input K tile_size_X tile_size_Y), its three output lines,
and the result checked per nonzero (--check-against) with the vector the CPU
oracle computes from the reference's own dense factors (0.1*drand48()), as the
reference's optional check does (sddmm.cu:133-141); --check repeats it against
the library's own CPU path."""
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
    cpu = oracle.sddmm_csr(d["row_ptr"].numpy(), cols, vals, W, H)
    expect = cpu.astype(np.float64).sum()
    vec = tmp_path / "oracle.f32"
    cpu.tofile(vec)
    for extra, tx, ty in (([], 192, 50000), (["--kernel", "row"], 0, 0), (["--kernel", "lds"], 64, 32),
                          (["--kernel", "panel", "--ref-order"], 32, 64), (["--kernel", "hybrid", "--check"], 0, 0)):
        dump = tmp_path / "out.f32"
        r = subprocess.run([CLI, str(mtx), str(K), str(tx), str(ty), "--json", "--runs", "3", "--check-against", str(vec),
                            "--dump-out", str(dump)] + extra, capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stderr + r.stdout
        out = r.stdout
        assert re.search(r"diff values in CPU and GPU: 0 ", out), out
        got = np.fromfile(dump, np.float32)
        assert got.shape == cpu.shape and np.all(np.abs(got - cpu) <= 1e-5 * np.sqrt(K) * np.abs(cpu) + 1e-6)
        if "--ref-order" in extra:
            assert re.search(r"Tilesize: X = 64, tilesize: Y = \d+", out), out
        if "--check" in extra:
            assert "Time for CPU SDDMM with K = 64" in out
        m = re.search(r"Matrix info:\s+rows: (\d+), cols: (\d+), nnz: (\d+)", out)
        assert m and tuple(map(int, m.groups())) == (d["n_rows"], d["n_cols"], d["nnz"])
        assert re.search(r"Tilesize: X = \d+, tilesize: Y = \d+, TB: \d+", out)
        m = re.search(r"Time for SDDMM with K = (\d+) : ([0-9.eE+-]+) ms", out)
        assert m and int(m.group(1)) == K and float(m.group(2)) > 0
        js = json.loads([ln for ln in out.splitlines() if ln.startswith("{")][0])
        assert js["nnz"] == d["nnz"] and js["K"] == K
        assert js["mismatches"] == 0 and js["max_rel"] <= 1e-5 * np.sqrt(K)
        assert abs(js["checksum"] - expect) <= 1e-5 * np.sqrt(K) * abs(expect) + 1e-6, (js["checksum"], expect)
    # a permuted or perturbed result must be caught per nonzero although its checksum is the same
    bad = cpu.copy(); bad[[3, 7]] = bad[[7, 3]]
    bad.tofile(vec)
    r = subprocess.run([CLI, str(mtx), str(K), "0", "0", "--check-against", str(vec)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and re.search(r"diff values in CPU and GPU: [12] ", r.stdout), r.stdout


def test_cli_column_sorted_input_and_errors(oracle, tmp_path):
    rng = np.random.default_rng(5)
    n, m = 60, 90
    keys = np.unique(rng.integers(0, n * m, 700))
    rows, cols = (keys // m).astype(np.int32), (keys % m).astype(np.int32)
    order = np.lexsort((rows, cols))  # column-sorted file, as the reference's conversion expects
    vals = rng.random(len(keys)).astype(np.float32) + 0.5
    p = tmp_path / "colsorted.mtx"
    capi.Coo.from_arrays(n, m, rows[order], cols[order], vals[order]).write_mtx(p)
    t_r, t_c, t_v, rp = oracle.transpose_sort(rows[order], cols[order], vals[order], m)
    W = oracle.initial(m, 32); H = oracle.initial(n, 32)
    cpu = oracle.sddmm_csr(rp, t_c, t_v, W, H)
    vec = tmp_path / "oracle_t.f32"
    cpu.tofile(vec)
    r = subprocess.run([CLI, str(p), "32", "16", "8", "--transpose", "--json", "--check-against", str(vec)], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 0, r.stderr + r.stdout
    assert f"rows: {m}, cols: {n}, nnz: {len(keys)}" in r.stdout
    js = json.loads([ln for ln in r.stdout.splitlines() if ln.startswith("{")][0])
    assert js["mismatches"] == 0
    # errors: missing file, bad K
    r = subprocess.run([CLI, str(tmp_path / "nope.mtx"), "32", "0", "0"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "cannot open" in r.stderr
    r = subprocess.run([CLI, str(p), "0", "0", "0"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0
    r = subprocess.run([CLI], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "usage" in r.stderr


def test_cli_tile_size_y_shapes_the_row_ranges_of_a_wide_matrix(oracle, tmp_path):
    """A banded matrix with more column tiles than workgroups is walked in row ranges; the
    fourth positional sets their height, and the second output line prints the height in use."""
    d = synth.make(5, 2.0 ** -3, K=128)
    rows = d["row_ind"].numpy(); cols = d["col_ind"].numpy(); vals = d["val"].numpy()
    S = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], rows, cols, vals)
    mtx = tmp_path / "banded.bin"
    S.write_bin(mtx)
    K = 128
    W = oracle.initial(d["n_rows"], K); H = oracle.initial(d["n_cols"], K)
    cpu = oracle.sddmm_csr(d["row_ptr"].numpy(), cols, vals, W, H)
    vec = tmp_path / "oracle.f32"
    cpu.tofile(vec)
    env = dict(os.environ, SDDMM_TILE_RUNS="2")
    seen = {}
    for ty in (0, 2048, 512):
        r = subprocess.run([CLI, str(mtx), str(K), "0", str(ty), "--no-plan-file", "--check-against", str(vec)], capture_output=True,
                           text=True, timeout=300, env=env)
        assert r.returncode == 0, r.stderr + r.stdout
        assert re.search(r"diff values in CPU and GPU: 0 ", r.stdout), r.stdout
        m = re.search(r"Tilesize: X = (\d+), tilesize: Y = (\d+), TB: (\d+)", r.stdout)
        assert m, r.stdout
        seen[ty] = int(m.group(2))
        if ty:
            # (ranges hold equal shares of the nonzeros: the clipped rows at the matrix edges make the outer ones taller)
            assert 0.9 * ty <= seen[ty] <= 1.7 * ty, (ty, seen)
            assert "is not used by this plan" not in r.stderr
    assert seen[0] > 2 * seen[2048] > 2 * seen[512], seen
    # a plan that cuts the rows into one block per die says that it does not use the value
    d3 = synth.make(3, 0.05, K=128)
    S3 = capi.Coo.from_arrays(d3["n_rows"], d3["n_cols"], d3["row_ind"].numpy(), d3["col_ind"].numpy(), d3["val"].numpy())
    p3 = tmp_path / "rec.bin"
    S3.write_bin(p3)
    r = subprocess.run([CLI, str(p3), "128", "0", "64", "--no-plan-file"], capture_output=True, text=True, timeout=300,
                       env=dict(os.environ, SDDMM_SPLIT_MIN_NNZ="0", SDDMM_TILE_FEW_BLOCKS="0"))
    assert r.returncode == 0, r.stderr + r.stdout
    assert "tile_size_Y = 64 is not used by this plan" in r.stderr, r.stderr


def test_cli_on_a_generated_matrix():
    """--gen: the tool makes the benchmark shape itself (no input file) and checks the device result per nonzero
    against the library's CPU path."""
    r = subprocess.run([CLI, "recommender", "128", "0", "0", "--gen", "3:0.02", "--check", "--json"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr + r.stdout
    m = re.search(r"Matrix info:  rows: (\d+), cols: (\d+), nnz: (\d+)", r.stdout)
    assert m and int(m.group(1)) == int(480189 * 0.02) and int(m.group(3)) > 100000
    assert re.search(r"diff values in CPU and GPU: 0 ", r.stdout), r.stdout
    r = subprocess.run([CLI, "x", "32", "0", "0", "--gen", "9"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "config must be 1..5" in r.stderr

