"""Host-side logic of libsddmm_hip.so (no GPU needed): the C ABI exports what
include/sddmm.h declares, the Matrix Market reader, the sorts, CSR builders,
the tiling pass (against the oracle's restatement of rewrite_matrix_1D and the
reference header where built) and the error behaviour."""
import ctypes
import os
import re

import numpy as np
import pytest
import scipy.sparse as sp

from sddmm_gpu_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def rand_coo(rng, n_rows, n_cols, nnz, sort=True):
    keys = np.unique(rng.integers(0, n_rows * n_cols, nnz))
    if not sort:
        keys = rng.permutation(keys)
    return (keys // n_cols).astype(np.int32), (keys % n_cols).astype(np.int32)


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "sddmm.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(sddmm_[a-z_0-9]+)\s*\(", hdr))
    assert len(declared) >= 20
    L = ctypes.CDLL(capi.LIB_PATH)
    for name in declared:
        assert hasattr(L, name), f"{name} declared in sddmm.h but not exported"
    assert declared == set(capi.SIGNATURES), declared ^ set(capi.SIGNATURES)
    assert b"gfx950" in capi.lib().sddmm_version()


def test_read_mtx_variants(tmp_path, oracle):
    body = "3 4 4\n1 1 0.5\n3 2 7e-1\n2 4 -2\n3 4 1\n"
    files = {
        "banner": "%%MatrixMarket matrix coordinate real general\n% a comment\n%another\n" + body,
        "headerless": body,
        "crlf": ("%%MatrixMarket matrix coordinate real general\n" + body).replace("\n", "\r\n"),
        "blank_lines": "%%MatrixMarket matrix coordinate real general\n\n" + body.replace("\n", "\n\n"),
        "integer": "%%MatrixMarket matrix coordinate integer general\n3 4 2\n1 2 3\n2 1 -4\n",
    }
    for name, text in files.items():
        p = tmp_path / f"{name}.mtx"
        p.write_text(text)
        S = capi.Coo.read_mtx(p)
        n, m, nnz, is_sorted = S.info()
        rows, cols, vals = S.arrays()
        if name == "integer":
            assert (n, m, nnz) == (3, 4, 2) and vals.tolist() == [3.0, -4.0]
            continue
        assert (n, m, nnz) == (3, 4, 4), name
        assert rows.tolist() == [0, 2, 1, 2] and cols.tolist() == [0, 1, 3, 3], name
        assert np.array_equal(vals, np.array([0.5, 0.7, -2, 1], np.float32)), name
        assert not is_sorted
        if name in ("banner", "headerless"):  # the reference's grammar reads the same triples
            on, om, orow, ocol, oval = oracle.parse_mtx(p)
            assert (on, om) == (n, m) and np.array_equal(orow, rows) and np.array_equal(ocol, cols) and np.array_equal(oval, vals)


def test_read_mtx_pattern_and_symmetric(tmp_path):
    p = tmp_path / "p.mtx"
    p.write_text("%%MatrixMarket matrix coordinate pattern general\n2 3 2\n1 3\n2 1\n")
    rows, cols, vals = capi.Coo.read_mtx(p).arrays()
    assert rows.tolist() == [0, 1] and cols.tolist() == [2, 0] and vals.tolist() == [1.0, 1.0]
    p = tmp_path / "s.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real symmetric\n3 3 3\n1 1 1\n2 1 2\n3 2 3\n")
    S = capi.Coo.read_mtx(p)
    S.sort_rows()
    rows, cols, vals = S.arrays()
    A = sp.coo_matrix((vals, (rows, cols)), shape=(3, 3)).toarray()
    assert np.array_equal(A, np.array([[1, 2, 0], [2, 0, 3], [0, 3, 0]], np.float32))


@pytest.mark.parametrize("text,code", [
    ("", capi.ERR_FORMAT),
    ("%%MatrixMarket matrix array real general\n2 2\n1\n2\n3\n4\n", capi.ERR_FORMAT),
    ("%%MatrixMarket matrix coordinate complex general\n1 1 1\n1 1 1 0\n", capi.ERR_FORMAT),
    ("%%MatrixMarket matrix coordinate real general\n2 2 3\n1 1 1\n2 2 2\n", capi.ERR_FORMAT),   # short
    ("%%MatrixMarket matrix coordinate real general\n2 2 1\n3 1 1\n", capi.ERR_RANGE),           # row 3 of 2
    ("%%MatrixMarket matrix coordinate real general\n2 2 1\n1 0 1\n", capi.ERR_RANGE),           # col 0
    ("%%MatrixMarket matrix coordinate real general\n2 2 1\n1 x 1\n", capi.ERR_FORMAT),
    ("%%MatrixMarket matrix coordinate real general\n2 2\n", capi.ERR_FORMAT),
])
def test_read_mtx_errors(tmp_path, text, code):
    p = tmp_path / "bad.mtx"
    p.write_text(text)
    with pytest.raises(capi.SddmmError) as e:
        capi.Coo.read_mtx(p)
    assert e.value.code == code
    assert "sddmm_read_mtx" in str(e.value)


def test_missing_file_and_bad_arguments(tmp_path):
    with pytest.raises(capi.SddmmError) as e:
        capi.Coo.read_mtx(tmp_path / "nope.mtx")
    assert e.value.code == capi.ERR_IO
    with pytest.raises(capi.SddmmError) as e:
        capi.Coo.from_arrays(2, 2, [0, 2], [0, 0])
    assert e.value.code == capi.ERR_RANGE
    S = capi.Coo.from_arrays(3, 3, [2, 0], [0, 1], [1.0, 2.0])
    for fn in (S.row_ptr, S.compress_rows, lambda: S.tiling(2, 2)):
        with pytest.raises(capi.SddmmError) as e:
            fn()
        assert e.value.code == capi.ERR_UNSORTED
    S.sort_rows()
    with pytest.raises(capi.SddmmError) as e:
        S.tiling(0, 2)
    assert e.value.code == capi.ERR_ARG


def test_large_file_parallel_parse_roundtrip(tmp_path):
    rng = np.random.default_rng(11)
    rows, cols = rand_coo(rng, 5000, 7000, 400_000, sort=False)
    vals = rng.standard_normal(len(rows)).astype(np.float32)
    S = capi.Coo.from_arrays(5000, 7000, rows, cols, vals)
    p = tmp_path / "big.mtx"
    S.write_mtx(p)
    assert os.path.getsize(p) > 4 << 20  # several parser chunks
    r2, c2, v2 = capi.Coo.read_mtx(p).arrays()
    assert np.array_equal(r2, rows) and np.array_equal(c2, cols) and np.array_equal(v2, vals)
    b = tmp_path / "big.bin"
    S.write_bin(b)
    T = capi.Coo.read_bin(b)
    r3, c3, v3 = T.arrays()
    assert np.array_equal(r3, rows) and np.array_equal(c3, cols) and np.array_equal(v3, vals)
    assert T.info() == S.info()
    b.write_bytes(b.read_bytes()[:100])
    with pytest.raises(capi.SddmmError) as e:
        capi.Coo.read_bin(b)
    assert e.value.code == capi.ERR_FORMAT


def test_sort_rows_is_stable_and_matches_scipy():
    rng = np.random.default_rng(12)
    n, m = 300, 200
    rows, cols = rand_coo(rng, n, m, 5000, sort=False)
    # add duplicates whose file order must be kept
    rows = np.concatenate([rows, rows[:50]]); cols = np.concatenate([cols, cols[:50]])
    vals = np.arange(len(rows), dtype=np.float32)
    S = capi.Coo.from_arrays(n, m, rows, cols, vals)
    assert not S.info()[3]
    S.sort_rows()
    r, c, v = S.arrays()
    order = np.lexsort((np.arange(len(rows)), cols, rows))  # stable (row, col)
    assert np.array_equal(r, rows[order]) and np.array_equal(c, cols[order]) and np.array_equal(v, vals[order])
    assert S.info()[3]
    rp = S.row_ptr()
    assert np.array_equal(rp, np.concatenate([[0], np.cumsum(np.bincount(rows, minlength=n))]))


def test_transpose_sort_matches_oracle(oracle):
    rng = np.random.default_rng(13)
    n, m = 40, 70
    rows, cols = rand_coo(rng, n, m, 600, sort=False)
    order = np.lexsort((rows, cols))  # a column-sorted file
    rows, cols = rows[order], cols[order]
    vals = rng.standard_normal(len(rows)).astype(np.float32)
    S = capi.Coo.from_arrays(n, m, rows, cols, vals)
    S.transpose_sort()
    assert S.info()[:2] == (m, n) and S.info()[3]
    r, c, v = S.arrays()
    o_r, o_c, o_v, rp = oracle.transpose_sort(rows, cols, vals, m)
    assert np.array_equal(r, o_r) and np.array_equal(c, o_c) and np.array_equal(v, o_v)
    assert np.array_equal(S.row_ptr(), rp)


def test_compress_rows_matches_make_csr(oracle):
    rng = np.random.default_rng(14)
    rows, cols = rand_coo(rng, 64, 64, 300)
    keep = rows % 5 != 2
    rows, cols = rows[keep], cols[keep]
    S = capi.Coo.from_arrays(64, 64, rows, cols)
    rp, holder = S.compress_rows()
    orp, oholder = oracle.make_csr(rows, 64)
    assert np.array_equal(rp, orp) and np.array_equal(holder, oholder)
    E = capi.Coo.from_arrays(5, 5, [], [])
    rp, holder = E.compress_rows()
    assert rp.tolist() == [0] and holder.tolist() == []
    assert E.row_ptr().tolist() == [0] * 6


def test_init_reference_matches_oracle(oracle):
    assert np.array_equal(capi.init_reference(7, 12), oracle.initial(7, 12))


def check_tiling_against(oracle_res, t, n_rows, actv):
    nt = oracle_res["n_tiles"]
    assert t["n_col_tiles"] == nt
    assert np.array_equal(t["tiled_ind"], oracle_res["tiled_ind"])
    assert np.array_equal(t["tile_ptr"], oracle_res["last_idx_tile"])
    assert np.array_equal(np.diff(t["active_ptr"]), oracle_res["n_actv_row"])
    assert t["max_active_rows"] == oracle_res["max_active_rows"]
    for j in range(nt):
        a0, a1 = t["active_ptr"][j], t["active_ptr"][j + 1]
        assert np.array_equal(t["active_row"][a0:a1], oracle_res["active_row"][j])
        nb = -(-int(a1 - a0) // actv)
        assert t["block_ptr"][j + 1] - t["block_ptr"][j] == nb
        assert np.array_equal(t["block_end"][t["block_ptr"][j]: t["block_ptr"][j + 1]], oracle_res["last_idx_block"][j][:nb])


@pytest.mark.parametrize("seed", range(8))
def test_tiling_matches_rewrite_matrix_1d(oracle, seed):
    rng = np.random.default_rng(200 + seed)
    n = int(rng.integers(3, 90)); m = int(rng.integers(3, 120))
    rows, cols = rand_coo(rng, n, m, int(rng.integers(1, n * m // 2 + 2)))
    if seed % 2:
        keep = rows % 4 != 1
        rows, cols = rows[keep], cols[keep]
    vals = rng.standard_normal(len(rows)).astype(np.float32)
    ts = int(rng.integers(1, m + 5)); actv = int(rng.integers(1, n + 3))
    S = capi.Coo.from_arrays(n, m, rows, cols, vals)
    t = S.tiling(ts, actv)
    check_tiling_against(oracle.rewrite_1d(n, m, rows, cols, vals, ts, actv), t, n, actv)
    # the tile-order copies the reference materialises follow from the permutation
    o = oracle.rewrite_1d(n, m, rows, cols, vals, ts, actv)
    assert np.array_equal(cols[t["tiled_ind"]], o["t_cols"]) and np.array_equal(vals[t["tiled_ind"]], o["t_vals"])


def test_tiling_known_answer_and_invariants(oracle):
    import json
    ka = json.load(open(os.path.join(ROOT, "tests", "golden", "tiling_known_answer.json")))
    S = capi.Coo.from_arrays(ka["n_rows"], ka["n_cols"], ka["rows"], ka["cols"], ka["vals"])
    t = S.tiling(ka["tile_size_x"], ka["actv_row_size"])
    assert t["tiled_ind"].tolist() == ka["tiled_ind"] and t["tile_ptr"].tolist() == ka["lastIdx_tile"]
    assert [t["active_row"][t["active_ptr"][j]: t["active_ptr"][j + 1]].tolist() for j in range(3)] == ka["active_row"]
    assert [int(t["block_end"][t["block_ptr"][j]]) for j in range(3)] == ka["first_block_end"]
    assert t["max_active_rows"] == ka["max_active_row"]
    # a larger, multi-threaded case: invariants
    rng = np.random.default_rng(21)
    n, m, X, Y = 3000, 5000, 192, 37
    rows, cols = rand_coo(rng, n, m, 600_000)
    S = capi.Coo.from_arrays(n, m, rows, cols)
    t = S.tiling(X, Y)
    perm = t["tiled_ind"]
    assert np.array_equal(np.sort(perm), np.arange(len(rows)))              # bijection
    tile_of = cols[perm] // X
    assert np.all(np.diff(tile_of) >= 0)                                     # tiles ascend
    assert np.array_equal(t["tile_ptr"], np.searchsorted(tile_of, np.arange(t["n_col_tiles"] + 1)))
    key = tile_of.astype(np.int64) * n * m + rows[perm].astype(np.int64) * m + cols[perm]
    assert np.all(np.diff(key) > 0)                                          # rows, then cols ascend inside a tile
    n_pairs = len(np.unique(tile_of.astype(np.int64) * n + rows[perm]))
    assert t["active_ptr"][-1] == n_pairs
    assert t["tile_ptr"][-1] == len(rows) and t["block_end"][-1] == len(rows)
    check_tiling_against(oracle.rewrite_1d(n, m, rows, cols, np.ones(len(rows), np.float32), X, Y), t, n, Y)


def test_tiling_matches_reference_header(oracle):
    if not oracle.have_ref():
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(22)
    n, m, X, Y = 50, 333, 20, 7
    rows, cols = rand_coo(rng, n, m, 3000)
    vals = rng.standard_normal(len(rows)).astype(np.float32)
    t = capi.Coo.from_arrays(n, m, rows, cols, vals).tiling(X, Y)
    ref, _ = oracle.ref_rewrite_1d(n, m, rows, cols, vals, X, Y)
    assert np.array_equal(t["tiled_ind"], ref["tiled_ind"])
    assert np.array_equal(t["tile_ptr"], ref["last_idx_tile"])
    assert np.array_equal(np.diff(t["active_ptr"]), ref["n_actv_row"])
    assert t["max_active_rows"] == ref["max_active_rows"]


@pytest.mark.parametrize("K,threads", [(1, 1), (7, 3), (32, 0), (100, 2)])
def test_sddmm_cpu_is_the_oracle_bit_for_bit(oracle, K, threads):
    # the library's own CPU path against the oracle's restatement of sddmm_CPU_CSR (sddmm.cu:153-177)
    rng = np.random.default_rng(K)
    n_rows, n_cols = 300, 211
    rows, cols = rand_coo(rng, n_rows, n_cols, 9000)
    vals = rng.uniform(-2, 2, len(rows)).astype(np.float32)
    W = rng.uniform(-1, 1, (n_rows, K)).astype(np.float32)
    H = rng.uniform(-1, 1, (n_cols, K)).astype(np.float32)
    S = capi.Coo.from_arrays(n_rows, n_cols, rows, cols, vals)
    got = S.cpu(K, W, H, threads)
    rp = S.row_ptr()
    want = oracle.sddmm_csr(rp, cols, vals, W, H)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_sddmm_cpu_config1_end_to_end(tmp_path, oracle):
    # BASELINE config 1 (4096 x 4096, 1 % density, K = 32) through the file reader, the sort and the CPU path
    from sddmm_gpu_amd import synth
    d = synth.make(1)
    S0 = capi.Coo.from_arrays(d["n_rows"], d["n_cols"], d["row_ind"].numpy(), d["col_ind"].numpy(), d["val"].numpy())
    path = tmp_path / "c1.mtx"
    S0.write_mtx(path)
    S = capi.Coo.read_mtx(path)
    S.sort_rows()
    r, c, v = S.arrays()
    assert np.array_equal(r, d["row_ind"].numpy()) and np.array_equal(c, d["col_ind"].numpy())
    W, H = d["W"].numpy(), d["H"].numpy()
    got = S.cpu(32, W, H)
    want = oracle.sddmm_csr(d["row_ptr"].numpy(), c, v, W, H)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    f64 = (W[r].astype(np.float64) * H[c].astype(np.float64)).sum(1) * v
    assert np.abs(got - f64).max() <= 1e-5 * np.sqrt(32) * np.abs(f64).max()


def test_cli_cpu_only_matches_oracle_per_nonzero(tmp_path, oracle):
    # the command-line tool without a GPU: reader, sort, CPU path, per-nonzero check against the oracle's vector
    import subprocess
    cli = os.path.join(ROOT, "sddmm_gpu_amd", "bin", "sddmm")
    rng = np.random.default_rng(11)
    rows, cols = rand_coo(rng, 200, 150, 3000, sort=False)
    vals = rng.uniform(0.5, 1.5, len(rows)).astype(np.float32)
    S = capi.Coo.from_arrays(200, 150, rows, cols, vals)
    mtx = tmp_path / "u.mtx"
    S.write_mtx(mtx)
    S.sort_rows()
    r, c, v = S.arrays()
    K = 32
    want = oracle.sddmm_csr(S.row_ptr(), c, v, oracle.initial(200, K), oracle.initial(150, K))
    vec = tmp_path / "want.f32"; want.tofile(vec)
    dump = tmp_path / "got.f32"
    p = subprocess.run([cli, str(mtx), str(K), "0", "0", "--cpu-only", "--cpu-threads", "2", "--check-against", str(vec),
                        "--dump-out", str(dump), "--json"], capture_output=True, text=True, timeout=60)
    assert p.returncode == 0, p.stderr + p.stdout
    assert "diff values in CPU and GPU: 0 " in p.stdout and "Time for CPU SDDMM with K = 32" in p.stdout
    assert np.array_equal(np.fromfile(dump, np.float32).view(np.uint32), want.view(np.uint32))
    (want * 1.001).astype(np.float32).tofile(vec)
    p = subprocess.run([cli, str(mtx), str(K), "0", "0", "--cpu-only", "--check-against", str(vec)], capture_output=True, text=True,
                       timeout=60)
    assert p.returncode == 1


def test_generated_benchmark_shapes(tmp_path, oracle):
    """sddmm_coo_generate: the five benchmark shapes made on the host.  Sorted, inside the matrix, without duplicates,
    the same for the same (config, scale, seed) whatever the number of threads, and with the statistics the shapes are
    defined by; the command-line tool reads one in place of a file and its CPU path agrees with the oracle on it."""
    import subprocess
    cli = os.path.join(ROOT, "sddmm_gpu_amd", "bin", "sddmm")
    want = {1: (1024, 1024, 10.24, None), 2: (375, 3104, 124.4, None), 3: (24009, 3973, 90.0, None), 4: (65536, 65536, 40.0, None),
            5: (65536, 65536, 62.6, 64)}
    scale = {1: 0.25, 2: 0.25, 3: 0.05, 4: 2.0 ** -6, 5: 2.0 ** -4}
    for cfg in range(1, 6):
        S = capi.Coo.generate(cfg, scale[cfg], seed=7)
        n_rows, n_cols, nnz, is_sorted = S.info()
        r, c, v = S.arrays()
        assert (n_rows, n_cols) == want[cfg][:2] and is_sorted and len(r) == nnz
        key = r.astype(np.int64) * n_cols + c
        assert np.all(np.diff(key) > 0) and r.min() >= 0 and r.max() < n_rows and c.min() >= 0 and c.max() < n_cols
        deg = np.bincount(r, minlength=n_rows)
        assert abs(deg.mean() / want[cfg][2] - 1) < 0.2, (cfg, deg.mean())
        if want[cfg][3]:
            assert deg.max() <= want[cfg][3]
        assert np.all(np.isfinite(v)) and v.min() > 0
        # (the thread count is read once per process: the one-thread run is the command-line tool's)
        one = tmp_path / ("one%d.bin" % cfg)
        p = subprocess.run([cli, "x", "4", "0", "0", "--gen", "%d:%r:7" % (cfg, scale[cfg]), "--cpu-only", "--save-bin", str(one)],
                           capture_output=True, text=True, timeout=120, env=dict(os.environ, SDDMM_NUM_THREADS="1"))
        assert p.returncode == 0, p.stderr + p.stdout
        r1, c1, v1 = capi.Coo.read_bin(one).arrays()
        assert np.array_equal(r, r1) and np.array_equal(c, c1) and np.array_equal(v, v1)
        r2, c2, _ = capi.Coo.generate(cfg, scale[cfg], seed=8).arrays()
        assert len(r2) != len(r) or not np.array_equal(c, c2)
    # what defines the shapes: the band; the heavy tails of the recommender's rows and columns; R-MAT's hubs
    r, c, v = capi.Coo.generate(5, 2.0 ** -4).arrays()
    assert np.abs(c.astype(np.int64) - r).max() <= 2048 and np.abs(c.astype(np.int64) - r).max() > 1900
    r, c, v = capi.Coo.generate(3, 0.05).arrays()
    deg = np.sort(np.bincount(r))[::-1]; pop = np.sort(np.bincount(c))[::-1]
    assert deg[: len(deg) // 100].sum() > 0.15 * len(r) and pop[: len(pop) // 10].sum() > 0.3 * len(c)
    assert set(np.unique(v)) == {1.0, 2.0, 3.0, 4.0, 5.0}
    r, c, v = capi.Coo.generate(4, 2.0 ** -6).arrays()
    assert np.bincount(r).max() > 100 * (len(r) / 65536) and np.all(v == 1.0)
    for bad in ((0, 1.0), (6, 1.0), (1, 0.0), (1, 1.5)):
        with pytest.raises(capi.SddmmError) as e:
            capi.Coo.generate(*bad)
        assert e.value.code == capi.ERR_ARG
    # the command-line tool on a generated matrix, CPU path, against the oracle's vector for the same matrix
    S = capi.Coo.generate(2, 0.25)
    n_rows, n_cols, nnz, _ = S.info()
    r, c, v = S.arrays()
    K = 16
    vec = tmp_path / "want.f32"
    oracle.sddmm_csr(S.row_ptr(), c, v, oracle.initial(n_rows, K), oracle.initial(n_cols, K)).tofile(vec)
    p = subprocess.run([cli, "generated", str(K), "0", "0", "--gen", "2:0.25", "--cpu-only", "--check-against", str(vec),
                        "--save-bin", str(tmp_path / "g.bin")], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr + p.stdout
    assert "Matrix info:  rows: %d, cols: %d, nnz: %d" % (n_rows, n_cols, nnz) in p.stdout
    assert "diff values in CPU and GPU: 0 " in p.stdout
    r3, c3, v3 = capi.Coo.read_bin(tmp_path / "g.bin").arrays()
    assert np.array_equal(r, r3) and np.array_equal(c, c3) and np.array_equal(v, v3)


def test_sddmm_cpu_errors():
    S = capi.Coo.from_arrays(3, 3, [2, 0], [0, 1])  # unsorted
    with pytest.raises(capi.SddmmError) as e:
        S.cpu(4, np.zeros((3, 4), np.float32), np.zeros((3, 4), np.float32))
    assert e.value.code == capi.ERR_UNSORTED
    S.sort_rows()
    assert capi.lib().sddmm_cpu(S.h, 0, None, None, None, 1) == capi.ERR_ARG
    E = capi.Coo.from_arrays(3, 3, [], [])
    assert len(E.cpu(4, np.zeros((3, 4), np.float32), np.zeros((3, 4), np.float32))) == 0


def test_plan_options_defaults_mean_choose():
    o = capi.PlanOptions.defaults()
    d = o.as_dict()
    assert d["kernel"] == capi.KERNEL_AUTO and d["tile_size_x"] == 0 and d["tile_size_y"] == 0 and d["ignore_env"] == 0
    assert all(v == -1 for k, v in d.items() if k not in ("kernel", "tile_size_x", "tile_size_y", "ignore_env")), d
    with pytest.raises(KeyError):
        capi.PlanOptions.defaults(no_such_field=1)


def test_plan_without_gpu_fails_loudly():
    n, arch = capi.device_info()
    if n > 0:
        pytest.skip("a GPU is present")
    S = capi.Coo.from_arrays(2, 2, [0, 1], [0, 1])
    with pytest.raises(capi.SddmmError) as e:
        S.plan(32)
    assert e.value.code == capi.ERR_HIP


def test_no_oracle_in_the_product():
    # the shipped package and library must not reach into oracle/
    for base, _, files in os.walk(os.path.join(ROOT, "sddmm_gpu_amd")):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".hpp", ".h")) or f == "Makefile":
                text = open(os.path.join(base, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(base, f)
