"""ctypes access to the CPU oracle (oracle/liboracle.so) and, when built, to
the reference's own util.h functions (oracle/_ref/libref_util.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never by the package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from ctypes import c_double, c_float, c_int, c_int32, c_int64, c_long, c_void_p, POINTER, byref

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle.so")
_REF = os.path.join(_HERE, "_ref", "libref_util.so")
_lib = None
_ref = None


def build():
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        _lib = C.CDLL(_LIB)
        _lib.oracle_sddmm_coo_timed.restype = c_double
        _lib.oracle_make_csr.restype = c_int64
        _lib.oracle_rewrite_1d.restype = c_int32
        _lib.oracle_max_threads.restype = c_int
    return _lib


def have_ref():
    return os.path.exists(_REF)


def ref():
    global _ref
    if _ref is None:
        _ref = C.CDLL(_REF)
        _ref.ref_make_CSR.restype = c_long
        _ref.ref_rewrite_matrix_1D.restype = c_int
    return _ref


def _p(a):
    return a.ctypes.data_as(c_void_p)


def _i32(a):
    return np.ascontiguousarray(a, np.int32)


def _f32(a):
    return np.ascontiguousarray(a, np.float32)


def max_threads():
    return lib().oracle_max_threads()


def sddmm_csr(row_ptr, col_ind, val, W, H, nthreads=0):
    """p[ind] = (sum_t W[r,t]*H[c,t]) * val[ind], sequential fp32 sum."""
    row_ptr, col_ind, val, W, H = _i32(row_ptr), _i32(col_ind), _f32(val), _f32(W), _f32(H)
    n_rows = len(row_ptr) - 1
    k = W.shape[1]
    out = np.empty(len(col_ind), np.float32)
    lib().oracle_sddmm_csr(c_int64(n_rows), _p(row_ptr), _p(col_ind), _p(val), c_int32(k), _p(W), _p(H), _p(out),
                           c_int(nthreads))
    return out


def sddmm_residual_csr(row_ptr, col_ind, val, W, H, nthreads=0):
    """p[ind] = val[ind] - (sum_t W[r,t]*H[c,t]), sequential fp32 sum."""
    row_ptr, col_ind, val, W, H = _i32(row_ptr), _i32(col_ind), _f32(val), _f32(W), _f32(H)
    n_rows = len(row_ptr) - 1
    k = W.shape[1]
    out = np.empty(len(col_ind), np.float32)
    lib().oracle_sddmm_residual_csr(c_int64(n_rows), _p(row_ptr), _p(col_ind), _p(val), c_int32(k), _p(W), _p(H), _p(out),
                                    c_int(nthreads))
    return out


def sddmm_coo(row_ind, col_ind, val, W, H, nthreads=0, apply_val=True, timed=False):
    row_ind, col_ind, val, W, H = _i32(row_ind), _i32(col_ind), _f32(val), _f32(W), _f32(H)
    k = W.shape[1]
    out = np.empty(len(col_ind), np.float32)
    args = (c_int64(len(col_ind)), _p(row_ind), _p(col_ind), _p(val), c_int32(k), _p(W), _p(H), _p(out),
            c_int(nthreads), c_int(1 if apply_val else 0))
    if timed:
        return out, lib().oracle_sddmm_coo_timed(*args)
    lib().oracle_sddmm_coo(*args)
    return out


def sddmm_f64(row_ind, col_ind, val, W, H):
    """(exact-ish product in fp64, conditioning term |val| * sum_t |w_t h_t|)."""
    row_ind, col_ind, val, W, H = _i32(row_ind), _i32(col_ind), _f32(val), _f32(W), _f32(H)
    k = W.shape[1]
    out = np.empty(len(col_ind), np.float64)
    absp = np.empty(len(col_ind), np.float64)
    lib().oracle_sddmm_f64(c_int64(len(col_ind)), _p(row_ind), _p(col_ind), _p(val), c_int32(k), _p(W), _p(H), _p(out),
                           _p(absp))
    return out, absp


def row_softmax(row_ptr, x):
    """Row-wise softmax over the stored entries (accumulated in fp64, rounded once)."""
    row_ptr, x = _i32(row_ptr), _f32(x)
    out = np.zeros(len(x), np.float32)
    lib().oracle_row_softmax(c_int64(len(row_ptr) - 1), _p(row_ptr), _p(x), _p(out))
    return out


def spmm_csr(row_ptr, col_ind, x, H, with_abs=False):
    """Y[r,:] = sum_p x[p] * H[col_p,:], sequential fp32; with_abs: also sum |x*h| in fp64."""
    row_ptr, col_ind, x, H = _i32(row_ptr), _i32(col_ind), _f32(x), _f32(H)
    n_rows = len(row_ptr) - 1
    k = H.shape[1]
    Y = np.empty((n_rows, k), np.float32)
    absy = np.empty((n_rows, k), np.float64) if with_abs else None
    lib().oracle_spmm_csr(c_int64(n_rows), _p(row_ptr), _p(col_ind), _p(x), c_int32(k), _p(H), _p(Y),
                          _p(absy) if with_abs else None)
    return (Y, absy) if with_abs else Y


def make_csr(rows, n_rows):
    rows = _i32(rows)
    row_ptr = np.zeros(n_rows + 2, np.int32)
    holder = np.zeros(n_rows + 1, np.int32)
    n = lib().oracle_make_csr(_p(rows), c_int64(len(rows)), c_int64(n_rows), _p(row_ptr), _p(holder))
    return row_ptr[: n + 1].copy(), holder[:n].copy()


def _tiling_buffers(n_rows, n_cols, nnz, ts, actv):
    ntile = n_cols // ts + 1
    max_blk = n_rows // actv + 1
    return dict(t_rows=np.zeros(nnz + 1, np.int32), t_cols=np.zeros(nnz + 1, np.int32),
                t_vals=np.zeros(nnz + 1, np.float32), t_ind=np.zeros(nnz + 1, np.int32),
                active_row=np.full(n_rows * ntile + 1, -1, np.int32), n_actv_row=np.zeros(ntile + 1, np.int32),
                last_idx_tile=np.zeros(ntile + 2, np.int32),
                last_idx_block=np.full((ntile + 1) * max_blk + 1, -1, np.int32)), ntile, max_blk


def _tiling_result(b, n_rows, n_cols, nnz, ts, max_blk, ret):
    nt = (n_cols + ts - 1) // ts
    n_act = b["n_actv_row"][:nt].copy()
    return dict(n_tiles=nt, max_active_rows=int(ret), t_rows=b["t_rows"][:nnz].copy(), t_cols=b["t_cols"][:nnz].copy(),
                t_vals=b["t_vals"][:nnz].copy(), tiled_ind=b["t_ind"][:nnz].copy(), n_actv_row=n_act,
                last_idx_tile=b["last_idx_tile"][: nt + 1].copy(),
                active_row=[b["active_row"][j * n_rows: j * n_rows + n_act[j]].copy() for j in range(nt)],
                last_idx_block=[b["last_idx_block"][j * max_blk: (j + 1) * max_blk].copy() for j in range(nt)])


def rewrite_1d(n_rows, n_cols, rows, cols, vals, ts, actv):
    """Oracle restatement of rewrite_matrix_1D on a sorted COO."""
    rows, cols, vals = _i32(rows), _i32(cols), _f32(vals)
    nnz = len(rows)
    row_ptr, holder = make_csr(rows, n_rows)
    b, ntile, max_blk = _tiling_buffers(n_rows, n_cols, nnz, ts, actv)
    ret = lib().oracle_rewrite_1d(c_int64(n_rows), c_int64(n_cols), c_int64(nnz), _p(cols), _p(vals), _p(row_ptr),
                                  _p(holder), c_int64(len(holder)), c_int32(ts), c_int32(actv), _p(b["t_rows"]),
                                  _p(b["t_cols"]), _p(b["t_vals"]), _p(b["t_ind"]), _p(b["active_row"]),
                                  _p(b["n_actv_row"]), _p(b["last_idx_tile"]), _p(b["last_idx_block"]))
    return _tiling_result(b, n_rows, n_cols, nnz, ts, max_blk, ret)


def initial(n, k, closed_form=False):
    X = np.empty((n, k), np.float32)
    (lib().oracle_initial_closed_form if closed_form else lib().oracle_initial)(_p(X), c_int64(n), c_int32(k))
    return X


def transpose_sort(rows, cols, vals, n_cols):
    rows, cols, vals = _i32(rows), _i32(cols), _f32(vals)
    nnz = len(rows)
    o_r, o_c, o_v = np.empty(nnz, np.int32), np.empty(nnz, np.int32), np.empty(nnz, np.float32)
    rp = np.zeros(n_cols + 1, np.int32)
    lib().oracle_transpose_sort(_p(rows), _p(cols), _p(vals), c_int64(nnz), c_int64(n_cols), _p(o_r), _p(o_c), _p(o_v),
                                _p(rp))
    return o_r, o_c, o_v, rp


def parse_mtx(path):
    r, c, z = c_int64(), c_int64(), c_int64()
    rc = lib().oracle_parse_mtx(str(path).encode(), byref(r), byref(c), byref(z), None, None, None)
    if rc:
        raise ValueError(f"oracle_parse_mtx failed with {rc}")
    rows, cols, vals = np.empty(z.value, np.int32), np.empty(z.value, np.int32), np.empty(z.value, np.float32)
    rc = lib().oracle_parse_mtx(str(path).encode(), byref(r), byref(c), byref(z), _p(rows), _p(cols), _p(vals))
    if rc:
        raise ValueError(f"oracle_parse_mtx failed with {rc}")
    return r.value, c.value, rows, cols, vals


# ---- the reference's own util.h, when oracle/_ref is built ----

def ref_make_csr(rows, cols, vals, n_rows):
    nnz = len(rows)
    rows_p = np.concatenate([_i32(rows), np.array([-1], np.int32)])
    cols_p = np.concatenate([_i32(cols), np.array([2**30], np.int32)])
    vals_p = np.concatenate([_f32(vals), np.zeros(1, np.float32)])
    row_ptr = np.full(n_rows + 2, nnz, np.int32)
    holder = np.zeros(n_rows + 1, np.int32)
    n = ref().ref_make_CSR(_p(rows_p), _p(cols_p), _p(vals_p), c_long(nnz), c_long(n_rows), _p(row_ptr), _p(holder))
    return row_ptr, holder, int(n)


def ref_rewrite_1d(n_rows, n_cols, rows, cols, vals, ts, actv):
    """rewrite_matrix_1D of the reference, run on padded copies (it reads one
    element past the arrays and row_ptr entries past the last non-empty row)."""
    nnz = len(rows)
    row_ptr, holder, n_holder = ref_make_csr(rows, cols, vals, n_rows)
    rows_p = np.concatenate([_i32(rows), np.array([-1], np.int32)])
    cols_p = np.concatenate([_i32(cols), np.array([2**30], np.int32)])
    vals_p = np.concatenate([_f32(vals), np.zeros(1, np.float32)])
    b, ntile, max_blk = _tiling_buffers(n_rows, n_cols, nnz, ts, actv)
    nt_out, mb_out = c_int(), c_int()
    ret = ref().ref_rewrite_matrix_1D(c_long(n_rows), c_long(n_cols), c_long(nnz), _p(rows_p), _p(cols_p), _p(vals_p),
                                      _p(row_ptr), _p(holder), c_int(ts), c_int(actv), _p(b["t_rows"]), _p(b["t_cols"]),
                                      _p(b["t_vals"]), _p(b["t_ind"]), _p(b["active_row"]), _p(b["n_actv_row"]),
                                      _p(b["last_idx_tile"]), _p(b["last_idx_block"]), byref(nt_out), byref(mb_out))
    assert nt_out.value == ntile and mb_out.value == max_blk
    return _tiling_result(b, n_rows, n_cols, nnz, ts, max_blk, ret), n_holder


def ref_initial(n, k):
    X = np.empty((n, k), np.float32)
    ref().ref_initial(_p(X), c_long(n), c_int(k))
    return X
