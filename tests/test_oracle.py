"""Pins the CPU oracle (oracle/sddmm_oracle.c): closed forms, fp64 brute force,
library routines, the known answers obtained from the reference's own util.h,
and -- where oracle/_ref is built -- that header itself on random inputs."""
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def rand_sorted_coo(rng, n_rows, n_cols, nnz):
    keys = np.unique(rng.integers(0, n_rows * n_cols, nnz))
    return (keys // n_cols).astype(np.int32), (keys % n_cols).astype(np.int32)


def row_ptr_of(rows, n_rows):
    return np.concatenate([[0], np.cumsum(np.bincount(rows, minlength=n_rows))]).astype(np.int32)


# ----------------------------------------------------------------- SDDMM ---

def test_all_ones_gives_k_times_val(oracle):
    rng = np.random.default_rng(0)
    rows, cols = rand_sorted_coo(rng, 37, 53, 400)
    val = rng.random(len(rows), dtype=np.float32) + 0.5
    for K in (1, 7, 32, 100):
        W = np.ones((37, K), np.float32)
        H = np.ones((53, K), np.float32)
        out = oracle.sddmm_csr(row_ptr_of(rows, 37), cols, val, W, H)
        assert np.array_equal(out, np.float32(K) * val)
        assert np.array_equal(oracle.sddmm_coo(rows, cols, val, W, H), out)


def test_k1_is_a_plain_product(oracle):
    rng = np.random.default_rng(1)
    rows, cols = rand_sorted_coo(rng, 20, 30, 200)
    val = rng.standard_normal(len(rows)).astype(np.float32)
    W = rng.standard_normal((20, 1)).astype(np.float32)
    H = rng.standard_normal((30, 1)).astype(np.float32)
    expect = (W[rows, 0] * H[cols, 0]) * val  # (0 + w*h) * val in fp32
    assert np.array_equal(oracle.sddmm_csr(row_ptr_of(rows, 20), cols, val, W, H), expect)


def test_one_hot_h_picks_a_w_entry(oracle):
    # H[c] = e_{j(c)}: out = val * W[r, j(c)] exactly (all other terms are +0)
    rng = np.random.default_rng(2)
    K = 16
    rows, cols = rand_sorted_coo(rng, 25, 40, 300)
    val = rng.standard_normal(len(rows)).astype(np.float32)
    W = rng.standard_normal((25, K)).astype(np.float32)
    j = rng.integers(0, K, 40)
    H = np.zeros((40, K), np.float32)
    H[np.arange(40), j] = 1.0
    expect = W[rows, j[cols]] * val
    assert np.array_equal(oracle.sddmm_csr(row_ptr_of(rows, 25), cols, val, W, H), expect)
    # and a transposed-operand mistake would show: W one-hot instead
    out2 = oracle.sddmm_csr(row_ptr_of(rows, 25), cols, val, W, H * 2)
    assert np.array_equal(out2, expect * 2)


def test_dense_s_equals_gemm(oracle):
    # S fully dense with val = 1: the result is W @ H.T (library routine)
    rng = np.random.default_rng(3)
    n, m, K = 23, 31, 48
    W = rng.standard_normal((n, K)).astype(np.float32)
    H = rng.standard_normal((m, K)).astype(np.float32)
    rows = np.repeat(np.arange(n, dtype=np.int32), m)
    cols = np.tile(np.arange(m, dtype=np.int32), n)
    out = oracle.sddmm_csr(row_ptr_of(rows, n), cols, np.ones(n * m, np.float32), W, H).reshape(n, m)
    ref = W.astype(np.float64) @ H.astype(np.float64).T
    absref = np.abs(W).astype(np.float64) @ np.abs(H).astype(np.float64).T
    assert np.all(np.abs(out - ref) <= K * 2.0 ** -24 * absref * 1.01)
    # n != m on purpose: swapped row/column roles cannot reproduce this matrix
    assert out.shape == ref.shape == (n, m)


def test_fp64_brute_force_and_sequential_order(oracle):
    rng = np.random.default_rng(4)
    n, m, K = 12, 9, 33
    rows, cols = rand_sorted_coo(rng, n, m, 60)
    val = rng.standard_normal(len(rows)).astype(np.float32)
    W = rng.standard_normal((n, K)).astype(np.float32)
    H = rng.standard_normal((m, K)).astype(np.float32)
    out = oracle.sddmm_csr(row_ptr_of(rows, n), cols, val, W, H)
    # python restatement of the rounding sequence: fp32 product, fp32 running sum, * val last
    for i in range(len(rows)):
        sm = np.float32(0)
        for t in range(K):
            sm = np.float32(sm + np.float32(W[rows[i], t] * H[cols[i], t]))
        assert out[i] == np.float32(sm * val[i])
    dense = sp.coo_matrix((val.astype(np.float64), (rows, cols)), shape=(n, m)).toarray() * (W.astype(np.float64) @ H.astype(np.float64).T)
    f64, absp = oracle.sddmm_f64(rows, cols, val, W, H)
    assert np.allclose(f64, dense[rows, cols], rtol=1e-13, atol=0)
    assert np.all(np.abs(out - f64) <= (K + 1) * 2.0 ** -24 * absp * 1.01)


def test_power_of_two_scaling_and_shipping_form(oracle):
    rng = np.random.default_rng(5)
    rows, cols = rand_sorted_coo(rng, 30, 30, 250)
    val = rng.standard_normal(len(rows)).astype(np.float32)
    W = rng.standard_normal((30, 64)).astype(np.float32)
    H = rng.standard_normal((30, 64)).astype(np.float32)
    rp = row_ptr_of(rows, 30)
    base = oracle.sddmm_csr(rp, cols, val, W, H)
    assert np.array_equal(oracle.sddmm_csr(rp, cols, val, W * 4, H), base * 4)
    assert np.array_equal(oracle.sddmm_csr(rp, cols, val * 0.5, W, H), base * 0.5)
    # the shipping reference loop leaves out "* val" (sddmm.cu:192)
    noval = oracle.sddmm_coo(rows, cols, val, W, H, apply_val=False)
    assert np.array_equal(noval * val, oracle.sddmm_coo(rows, cols, val, W, H))
    assert np.array_equal(oracle.sddmm_coo(rows, cols, val, W, H, nthreads=3), base)


def test_residual_form_is_the_same_loop_with_another_last_operation(oracle):
    """val - dot: bit for bit val minus the (pinned) scaled form run with val = 1;
    closed form W = H = 1 -> val - K; fp64 brute force on a tiny case."""
    rng = np.random.default_rng(11)
    n_rows, n_cols, K = 37, 53, 24
    rows, cols = rand_sorted_coo(rng, n_rows, n_cols, 400)
    rp = row_ptr_of(rows, n_rows)
    val = rng.standard_normal(len(rows)).astype(np.float32)
    W = rng.standard_normal((n_rows, K)).astype(np.float32)
    H = rng.standard_normal((n_cols, K)).astype(np.float32)
    res = oracle.sddmm_residual_csr(rp, cols, val, W, H)
    dot = oracle.sddmm_csr(rp, cols, np.ones_like(val), W, H)
    assert np.array_equal(res, val - dot)
    f64 = val.astype(np.float64) - np.einsum("ij,ij->i", W[rows].astype(np.float64), H[cols].astype(np.float64))
    assert np.abs(res - f64).max() <= 1e-5 * np.sqrt(K) * np.abs(W[rows] * H[cols]).sum(1).max()
    ones = oracle.sddmm_residual_csr(rp, cols, val, np.ones_like(W), np.ones_like(H))
    assert np.array_equal(ones, val - np.float32(K))
    assert np.array_equal(oracle.sddmm_residual_csr(rp, cols, val, W, H, nthreads=1), res)


def test_permuting_nonzeros_permutes_outputs(oracle):
    rng = np.random.default_rng(6)
    rows, cols = rand_sorted_coo(rng, 40, 50, 500)
    val = rng.standard_normal(len(rows)).astype(np.float32)
    W = rng.standard_normal((40, 24)).astype(np.float32)
    H = rng.standard_normal((50, 24)).astype(np.float32)
    base = oracle.sddmm_coo(rows, cols, val, W, H)
    perm = rng.permutation(len(rows))
    assert np.array_equal(oracle.sddmm_coo(rows[perm], cols[perm], val[perm], W, H), base[perm])


# ------------------------------------------------------ host transforms ---

def test_tiling_known_answer_from_reference_header(oracle):
    # golden/tiling_known_answer.json: inputs and outputs recorded from the
    # reference's util.h (make_CSR + rewrite_matrix_1D) on a 4x5 matrix
    ka = json.load(open(os.path.join(GOLDEN, "tiling_known_answer.json")))
    rp, holder = oracle.make_csr(ka["rows"], ka["n_rows"])
    assert rp.tolist() == ka["row_ptr"] and holder.tolist() == ka["row_holder"]
    r = oracle.rewrite_1d(ka["n_rows"], ka["n_cols"], ka["rows"], ka["cols"], ka["vals"], ka["tile_size_x"], ka["actv_row_size"])
    assert r["n_tiles"] == ka["ntile_c"]
    assert r["t_rows"].tolist() == ka["tiled_rows"] and r["t_cols"].tolist() == ka["tiled_cols"]
    assert r["t_vals"].tolist() == ka["tiled_vals"] and r["tiled_ind"].tolist() == ka["tiled_ind"]
    assert r["last_idx_tile"].tolist() == ka["lastIdx_tile"]
    assert [a.tolist() for a in r["active_row"]] == ka["active_row"]
    assert r["n_actv_row"].tolist() == ka["n_actv_row"]
    assert [int(b[0]) for b in r["last_idx_block"]] == ka["first_block_end"]
    assert r["max_active_rows"] == ka["max_active_row"]


def test_initial_known_values_and_closed_form(oracle):
    ka = json.load(open(os.path.join(GOLDEN, "initial_known_answer.json")))
    X = oracle.initial(3, 8)
    assert np.allclose(X.ravel()[:8], ka["first8"], rtol=1e-7, atol=0)
    assert np.array_equal(X, oracle.initial(3, 8, closed_form=True))
    # srand48(0) inside: W and H share a prefix (util.h:76)
    assert np.array_equal(oracle.initial(5, 4).ravel()[:12], oracle.initial(3, 4).ravel())
    assert X.min() >= 0 and X.max() < 0.1


def test_transpose_sort_matches_scipy(oracle):
    rng = np.random.default_rng(7)
    n, m = 17, 29
    keys = rng.permutation(np.unique(rng.integers(0, n * m, 200)))
    rows, cols = (keys // m).astype(np.int32), (keys % m).astype(np.int32)
    vals = rng.standard_normal(len(keys)).astype(np.float32)
    o_r, o_c, o_v, rp = oracle.transpose_sort(rows, cols, vals, m)
    A = sp.coo_matrix((vals, (rows, cols)), shape=(n, m)).T.tocsr()
    A.sort_indices()
    assert np.array_equal(rp, A.indptr) and np.array_equal(o_c, A.indices) and np.array_equal(o_v, A.data)
    assert np.array_equal(o_r, np.repeat(np.arange(m), np.diff(A.indptr)))


def test_parse_mtx_reference_grammar(oracle, tmp_path):
    p = tmp_path / "a.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n% comment\n3 4 3\n1 1 0.5\n2 4 -2\n3 2 7e-1\n")
    n, m, rows, cols, vals = oracle.parse_mtx(p)
    assert (n, m) == (3, 4) and rows.tolist() == [0, 1, 2] and cols.tolist() == [0, 3, 1]
    assert np.array_equal(vals, np.array([0.5, -2, 0.7], np.float32))


# ------------------------------------------- the reference's own header ---

@pytest.mark.parametrize("seed", range(6))
def test_restatements_match_reference_header(oracle, seed):
    if not oracle.have_ref():
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(100 + seed)
    n = int(rng.integers(5, 60)); m = int(rng.integers(5, 80))
    rows, cols = rand_sorted_coo(rng, n, m, int(rng.integers(1, n * m // 2)))
    if seed % 2:  # leave some rows empty
        keep = rows % 3 != 1
        rows, cols = rows[keep], cols[keep]
    vals = rng.standard_normal(len(rows)).astype(np.float32)
    ts = int(rng.integers(1, m + 3)); actv = int(rng.integers(1, n + 2))
    rp_ref, holder_ref, nh = oracle.ref_make_csr(rows, cols, vals, n)
    rp, holder = oracle.make_csr(rows, n)
    assert nh == len(holder) and np.array_equal(rp, rp_ref[: nh + 1]) and np.array_equal(holder, holder_ref[:nh])
    mine = oracle.rewrite_1d(n, m, rows, cols, vals, ts, actv)
    ref, _ = oracle.ref_rewrite_1d(n, m, rows, cols, vals, ts, actv)
    for k in ("t_rows", "t_cols", "t_vals", "tiled_ind", "n_actv_row", "last_idx_tile"):
        assert np.array_equal(mine[k], ref[k]), k
    assert mine["max_active_rows"] == ref["max_active_rows"]
    for j in range(mine["n_tiles"]):
        assert np.array_equal(mine["active_row"][j], ref["active_row"][j])
        nb = -(-int(mine["n_actv_row"][j]) // actv)
        # slot 0 of tiles >= 1 is where the reference's stray first-block write lands (util.h:289-292)
        lo = 1 if (j >= 1 and nb > 1) else 0
        if nb and not (j >= 1 and nb == 1):
            assert np.array_equal(mine["last_idx_block"][j][lo:nb], ref["last_idx_block"][j][lo:nb]), j
    assert np.array_equal(oracle.initial(n, 7), oracle.ref_initial(n, 7))


# ------------------------------------------------- row softmax and SpMM ---

def test_row_softmax_closed_forms(oracle):
    rng = np.random.default_rng(3)
    rows, cols = rand_sorted_coo(rng, 60, 80, 900)
    rp = row_ptr_of(rows, 60)
    deg = np.diff(rp)
    # equal logits -> 1 / row length, whatever the common value
    for c in (0.0, -7.5, 88.0):
        out = oracle.row_softmax(rp, np.full(len(rows), c, np.float32))
        assert np.allclose(out, 1.0 / deg[rows], rtol=1e-7, atol=0)
    x = rng.normal(0, 3, len(rows)).astype(np.float32)
    out = oracle.row_softmax(rp, x)
    sums = np.bincount(rows, weights=out.astype(np.float64), minlength=60)
    assert np.allclose(sums[deg > 0], 1.0, atol=1e-6) and np.all(sums[deg == 0] == 0)
    # shift invariance per row (a dropped max or a wrong sign in the exponent fails here) and order preservation
    shift = rng.integers(-20, 20, 60).astype(np.float32)
    assert np.allclose(oracle.row_softmax(rp, x + shift[rows]), out, rtol=2e-6, atol=1e-12)
    r = int(np.argmax(deg)); seg = slice(rp[r], rp[r + 1])
    assert np.array_equal(np.argsort(x[seg], kind="stable"), np.argsort(out[seg], kind="stable"))
    # one dominant logit -> 1 for it, 0 for the rest; two entries -> the logistic function
    x2 = x.copy(); x2[rp[r]] = 1e4
    o2 = oracle.row_softmax(rp, x2)
    assert o2[rp[r]] == 1.0 and np.all(o2[rp[r] + 1:rp[r + 1]] == 0)
    two = oracle.row_softmax(np.array([0, 2], np.int32), np.array([0.3, -1.1], np.float32))
    assert np.allclose(two, [1 / (1 + np.exp(-1.4)), 1 / (1 + np.exp(1.4))], rtol=1e-6)


def test_row_softmax_matches_fp64_brute_force(oracle):
    rng = np.random.default_rng(4)
    rows, cols = rand_sorted_coo(rng, 25, 3000, 20000)
    rp = row_ptr_of(rows, 25)
    x = rng.normal(0, 5, len(rows)).astype(np.float32)
    out = oracle.row_softmax(rp, x)
    for r in range(25):
        seg = x[rp[r]:rp[r + 1]].astype(np.float64)
        if len(seg):
            e = np.exp(seg - seg.max())
            assert np.allclose(out[rp[r]:rp[r + 1]], e / e.sum(), rtol=3e-7, atol=1e-37)


def test_spmm_matches_scipy_closed_forms_and_fp64(oracle):
    rng = np.random.default_rng(5)
    n, m = 70, 90
    rows, cols = rand_sorted_coo(rng, n, m, 1500)
    rp = row_ptr_of(rows, n)
    x = rng.normal(0, 1, len(rows)).astype(np.float32)
    for K in (1, 5, 32, 100):
        H = rng.normal(0, 1, (m, K)).astype(np.float32)
        Y, absy = oracle.spmm_csr(rp, cols, x, H, with_abs=True)
        A = sp.csr_matrix((x.astype(np.float64), cols, rp), shape=(n, m))
        ref = A @ H.astype(np.float64)
        assert np.all(np.abs(Y - ref) <= 1e-6 * np.sqrt(32) * absy + 1e-30)
        assert np.allclose(absy, abs(A) @ np.abs(H.astype(np.float64)))
        assert np.all(Y[np.diff(rp) == 0] == 0)  # rows without entries
    # one-hot H picks, per row, the sum of the entries whose column maps to that output column
    K = 8
    j = rng.integers(0, K, m)
    H = np.zeros((m, K), np.float32); H[np.arange(m), j] = 1.0
    xi = rng.integers(1, 6, len(rows)).astype(np.float32)  # small integers: every sum is exact
    Y = oracle.spmm_csr(rp, cols, xi, H)
    want = np.zeros((n, K)); np.add.at(want, (rows, j[cols]), xi)
    assert np.array_equal(Y, want.astype(np.float32))
    # all ones: the row sums, exactly
    Y = oracle.spmm_csr(rp, cols, xi, np.ones((m, 3), np.float32))
    assert np.array_equal(Y[:, 1], np.bincount(rows, weights=xi, minlength=n).astype(np.float32))
