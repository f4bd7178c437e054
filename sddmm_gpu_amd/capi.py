"""ctypes binding of include/sddmm.h (libsddmm_hip.so, built in-tree).

The library is the product; this module only declares its entry points and
wraps the opaque handles.  Loading fails loudly when the library has not been
built: there is no fallback path.
"""
from __future__ import annotations

import ctypes as C
import os
from ctypes import POINTER, byref, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_uint32, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsddmm_hip.so")

OK, ERR_ARG, ERR_IO, ERR_FORMAT, ERR_RANGE, ERR_UNSORTED, ERR_HIP, ERR_NOMEM = range(8)
KERNEL_AUTO, KERNEL_ROW_GATHER, KERNEL_LDS_TILE, KERNEL_PANEL, KERNEL_HYBRID, KERNEL_DENSE_BLOCK = 0, 1, 2, 3, 4, 5
EPILOGUE_SCALE, EPILOGUE_RESIDUAL = 0, 1
FORM_SOFTMAX = 0x100


class SddmmError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"sddmm error {code}: {msg}")
        self.code = code


class PlanInfo(C.Structure):
    _fields_ = [("n_rows", c_int64), ("n_cols", c_int64), ("nnz", c_int64), ("rows_touched", c_int64),
                ("cols_touched", c_int64), ("K", c_int32), ("tile_size_x", c_int32), ("tile_size_y", c_int32),
                ("k_slice", c_int32), ("n_col_tiles", c_int32), ("n_row_panels", c_int32), ("kernel", c_int32), ("n_launches", c_int32),
                ("lanes_per_nnz", c_int32), ("lds_bytes", c_int32), ("grid", c_int32), ("block", c_int32),
                ("n_blocks", c_int64), ("device_bytes", c_int64), ("class_nnz", c_int64 * 3), ("class_rows", c_int64 * 3), ("padded_positions", c_int64),
                ("short_batches", c_int64),
                ("plan_ms", c_double), ("dense_nnz", c_int64), ("dense_blocks", c_int64), ("matrix_nnz", c_int64),
                ("matrix_rows", c_int64), ("spmm_runs", c_int64)]

    def as_dict(self):
        return {f: (list(getattr(self, f)) if f.startswith("class_") else getattr(self, f)) for f, _ in self._fields_}


class PlanOptions(C.Structure):
    """sddmm_plan_options; PlanOptions.defaults(**fields) starts from sddmm_plan_options_init."""
    _fields_ = [(n, c_int32) for n in (
        "kernel", "tile_size_x", "tile_size_y", "k_slice", "tile_lanes", "tile_waves", "tile_assign", "tile_few_blocks",
        "tile_short_batches", "tile_deal", "tile_runs", "gather_lanes", "gather_padded", "gather_sink", "row_padded",
        "unpadded_tile", "dense_blocks", "dense_permille", "dense_rb_group", "fuse_slices", "matrix_rows", "matrix_permille", "matrix_waves", "spmm_stream", "ignore_env")] + [(n, c_int64) for n in (
        "gather_slab_cols", "gather_panel_rows", "dense_min_nnz", "panel_bytes", "short_row_max", "stage_factor", "split_min_nnz")]

    @classmethod
    def defaults(cls, **kw):
        o = cls()
        lib().sddmm_plan_options_init(byref(o))
        for k, v in kw.items():
            if k not in dict(cls._fields_):
                raise KeyError(k)
            setattr(o, k, v)
        return o

    def as_dict(self):
        return {f: getattr(self, f) for f, _ in self._fields_}


class LaunchProfile(C.Structure):
    _fields_ = [("kernel", c_int32), ("lanes_per_nnz", c_int32), ("k_slice", c_int32), ("n_kernel_launches", c_int32),
                ("nnz", c_int64), ("rows", c_int64), ("stream_positions", c_int64), ("ms", c_float)]


class TilingView(C.Structure):
    _fields_ = [("tile_size_x", c_int32), ("tile_size_y", c_int32), ("n_col_tiles", c_int32),
                ("max_active_rows", c_int32), ("nnz", c_int64), ("tile_ptr", POINTER(c_int32)),
                ("tiled_ind", POINTER(c_int32)), ("active_ptr", POINTER(c_int64)), ("active_row", POINTER(c_int32)),
                ("active_end", POINTER(c_int32)), ("block_ptr", POINTER(c_int64)), ("block_end", POINTER(c_int32))]


# every symbol include/sddmm.h declares: name -> (restype, argtypes)
SIGNATURES = {
    "sddmm_last_error": (c_char_p, []),
    "sddmm_version": (c_char_p, []),
    "sddmm_read_mtx": (c_int, [c_char_p, POINTER(c_void_p)]),
    "sddmm_write_mtx": (c_int, [c_void_p, c_char_p]),
    "sddmm_write_bin": (c_int, [c_void_p, c_char_p]),
    "sddmm_read_bin": (c_int, [c_char_p, POINTER(c_void_p)]),
    "sddmm_coo_generate": (c_int, [c_int32, C.c_double, C.c_uint64, POINTER(c_void_p)]),
    "sddmm_coo_create": (c_int, [c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, POINTER(c_void_p)]),
    "sddmm_coo_destroy": (None, [c_void_p]),
    "sddmm_coo_info": (c_int, [c_void_p, POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), POINTER(c_int)]),
    "sddmm_coo_arrays": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p)]),
    "sddmm_coo_sort_rows": (c_int, [c_void_p]),
    "sddmm_coo_transpose_sort": (c_int, [c_void_p]),
    "sddmm_coo_row_ptr": (c_int, [c_void_p, c_void_p]),
    "sddmm_coo_compress_rows": (c_int, [c_void_p, c_void_p, c_void_p, POINTER(c_int64)]),
    "sddmm_init_reference": (c_int, [c_void_p, c_int64, c_int32]),
    "sddmm_cpu": (c_int, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int32]),
    "sddmm_tiling_create": (c_int, [c_void_p, c_int32, c_int32, POINTER(c_void_p)]),
    "sddmm_tiling_get": (c_int, [c_void_p, POINTER(TilingView)]),
    "sddmm_tiling_destroy": (None, [c_void_p]),
    "sddmm_plan_create": (c_int, [c_void_p, c_int32, c_int32, c_int32, c_uint32, POINTER(c_void_p)]),
    "sddmm_plan_create_device": (c_int, [c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int32, c_int32, c_int32,
                                         c_uint32, POINTER(c_void_p)]),
    "sddmm_plan_options_init": (None, [POINTER(PlanOptions)]),
    "sddmm_plan_create_opt": (c_int, [c_void_p, c_int32, POINTER(PlanOptions), POINTER(c_void_p)]),
    "sddmm_plan_create_device_opt": (c_int, [c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int32, POINTER(PlanOptions),
                                             POINTER(c_void_p)]),
    "sddmm_plan_get_options": (c_int, [c_void_p, POINTER(PlanOptions)]),
    "sddmm_plan_save": (c_int, [c_void_p, c_char_p]),
    "sddmm_plan_load": (c_int, [c_char_p, c_void_p, c_int32, POINTER(PlanOptions), POINTER(c_void_p)]),
    "sddmm_plan_load_device": (c_int, [c_char_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int32, POINTER(PlanOptions),
                                       POINTER(c_void_p)]),
    "sddmm_plan_set_values": (c_int, [c_void_p, c_void_p, c_void_p]),
    "sddmm_plan_get_info": (c_int, [c_void_p, POINTER(PlanInfo)]),
    "sddmm_plan_destroy": (None, [c_void_p]),
    "sddmm_execute": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sddmm_execute_epilogue": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p]),
    "sddmm_execute_softmax": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sddmm_plan_workspace_bytes": (c_int, [c_void_p, POINTER(c_int64)]),
    "sddmm_execute_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_int64, c_void_p]),
    "sddmm_plan_spmm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "sddmm_row_softmax": (c_int, [c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sddmm_spmm_csr": (c_int, [c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p]),
    "sddmm_plan_launch_count": (c_int, [c_void_p, POINTER(c_int32)]),
    "sddmm_execute_profiled": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(LaunchProfile), c_int32]),
    "sddmm_gpu": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, POINTER(c_float)]),
    "sddmm_csr_noalloc": (c_int, [c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p,
                                  c_void_p, c_void_p]),
    "sddmm_copy_probe": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "sddmm_device_info": (c_int, [POINTER(c_int), c_char_p, c_int]),
}

_lib = None


def lib():
    """The loaded C library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `make -C sddmm_gpu_amd/csrc` "
                              "(or __graft_entry__.build()); there is no fallback implementation")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc):
    if rc != OK:
        raise SddmmError(rc, lib().sddmm_last_error().decode())


def _np_ptr(a):
    return a.ctypes.data_as(c_void_p)


class Coo:
    """Host-side sparse matrix handle (sddmm_coo)."""

    def __init__(self, handle):
        self.h = handle

    @classmethod
    def from_arrays(cls, n_rows, n_cols, rows, cols, vals=None):
        rows = np.ascontiguousarray(rows, dtype=np.int32)
        cols = np.ascontiguousarray(cols, dtype=np.int32)
        vp = None
        if vals is not None:
            vals = np.ascontiguousarray(vals, dtype=np.float32)
            vp = _np_ptr(vals)
        h = c_void_p()
        check(lib().sddmm_coo_create(n_rows, n_cols, len(rows), _np_ptr(rows), _np_ptr(cols), vp, byref(h)))
        return cls(h)

    @classmethod
    def read_mtx(cls, path):
        h = c_void_p()
        check(lib().sddmm_read_mtx(str(path).encode(), byref(h)))
        return cls(h)

    @classmethod
    def read_bin(cls, path):
        h = c_void_p()
        check(lib().sddmm_read_bin(str(path).encode(), byref(h)))
        return cls(h)

    @classmethod
    def generate(cls, config, scale=1.0, seed=None):
        """One of the five benchmark shapes, generated on the host (sddmm_coo_generate)."""
        h = c_void_p()
        check(lib().sddmm_coo_generate(config, float(scale), config if seed is None else seed, byref(h)))
        return cls(h)

    def write_mtx(self, path):
        check(lib().sddmm_write_mtx(self.h, str(path).encode()))

    def write_bin(self, path):
        check(lib().sddmm_write_bin(self.h, str(path).encode()))

    def info(self):
        r, c, n, s = c_int64(), c_int64(), c_int64(), c_int()
        check(lib().sddmm_coo_info(self.h, byref(r), byref(c), byref(n), byref(s)))
        return r.value, c.value, n.value, bool(s.value)

    def arrays(self):
        """Copies of (rows, cols, vals)."""
        _, _, nnz, _ = self.info()
        r, c, v = c_void_p(), c_void_p(), c_void_p()
        check(lib().sddmm_coo_arrays(self.h, byref(r), byref(c), byref(v)))
        if nnz == 0:
            return np.zeros(0, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32)
        rows = np.ctypeslib.as_array(C.cast(r, POINTER(c_int32)), (nnz,)).copy()
        cols = np.ctypeslib.as_array(C.cast(c, POINTER(c_int32)), (nnz,)).copy()
        vals = np.ctypeslib.as_array(C.cast(v, POINTER(c_float)), (nnz,)).copy()
        return rows, cols, vals

    def sort_rows(self):
        check(lib().sddmm_coo_sort_rows(self.h))

    def transpose_sort(self):
        check(lib().sddmm_coo_transpose_sort(self.h))

    def row_ptr(self):
        n_rows = self.info()[0]
        rp = np.empty(n_rows + 1, np.int32)
        check(lib().sddmm_coo_row_ptr(self.h, _np_ptr(rp)))
        return rp

    def compress_rows(self):
        n_rows = self.info()[0]
        rp = np.zeros(n_rows + 1, np.int32)
        rh = np.zeros(max(n_rows, 1), np.int32)
        n = c_int64()
        check(lib().sddmm_coo_compress_rows(self.h, _np_ptr(rp), _np_ptr(rh), byref(n)))
        return rp[: n.value + 1].copy(), rh[: n.value].copy()

    def tiling(self, tile_x, tile_y):
        h = c_void_p()
        check(lib().sddmm_tiling_create(self.h, tile_x, tile_y, byref(h)))
        try:
            v = TilingView()
            check(lib().sddmm_tiling_get(h, byref(v)))
            nt = v.n_col_tiles

            def arr(p, n, dt):
                return np.ctypeslib.as_array(p, (n,)).astype(dt, copy=True) if n else np.zeros(0, dt)

            active_ptr = arr(v.active_ptr, nt + 1, np.int64)
            block_ptr = arr(v.block_ptr, nt + 1, np.int64)
            return dict(tile_size_x=v.tile_size_x, tile_size_y=v.tile_size_y, n_col_tiles=nt,
                        max_active_rows=v.max_active_rows, nnz=v.nnz,
                        tile_ptr=arr(v.tile_ptr, nt + 1, np.int32), tiled_ind=arr(v.tiled_ind, v.nnz, np.int32),
                        active_ptr=active_ptr, active_row=arr(v.active_row, int(active_ptr[-1]), np.int32),
                        active_end=arr(v.active_end, int(active_ptr[-1]), np.int32), block_ptr=block_ptr,
                        block_end=arr(v.block_end, int(block_ptr[-1]), np.int32))
        finally:
            lib().sddmm_tiling_destroy(h)

    def plan(self, K, tile_x=0, tile_y=0, kernel=KERNEL_AUTO, options=None):
        h = c_void_p()
        if options is not None:
            check(lib().sddmm_plan_create_opt(self.h, K, byref(options), byref(h)))
        else:
            check(lib().sddmm_plan_create(self.h, K, tile_x, tile_y, kernel, byref(h)))
        return Plan(h)

    def load_plan(self, path, K, options=None):
        """A plan saved by Plan.save for this matrix, K and options (None: any options)."""
        h = c_void_p()
        check(lib().sddmm_plan_load(str(path).encode(), self.h, K, byref(options) if options is not None else None, byref(h)))
        return Plan(h)

    def cpu(self, K, W, H, n_threads=0):
        """The SDDMM on the host cores (sddmm_cpu): fp32, sequential sums, no GPU needed."""
        n_rows, n_cols, nnz, _ = self.info()
        W = np.ascontiguousarray(W, np.float32)
        H = np.ascontiguousarray(H, np.float32)
        assert W.size == n_rows * K and H.size == n_cols * K
        out = np.empty(nnz, np.float32)
        check(lib().sddmm_cpu(self.h, K, _np_ptr(W), _np_ptr(H), _np_ptr(out), n_threads))
        return out

    def close(self):
        if self.h:
            lib().sddmm_coo_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Plan:
    """Device execution plan handle (sddmm_plan).  Pointers passed to execute
    are raw device addresses (e.g. torch.Tensor.data_ptr())."""

    def __init__(self, handle, keep=None):
        self.h = handle
        self._keep = keep  # device arrays the plan borrows

    @classmethod
    def from_device_csr(cls, n_rows, n_cols, nnz, d_row_ptr, d_col_ind, K, tile_x=0, tile_y=0, kernel=KERNEL_AUTO,
                        keep=None, options=None):
        h = c_void_p()
        if options is not None:
            check(lib().sddmm_plan_create_device_opt(n_rows, n_cols, nnz, c_void_p(d_row_ptr), c_void_p(d_col_ind), K,
                                                     byref(options), byref(h)))
        else:
            check(lib().sddmm_plan_create_device(n_rows, n_cols, nnz, c_void_p(d_row_ptr), c_void_p(d_col_ind), K, tile_x,
                                                 tile_y, kernel, byref(h)))
        return cls(h, keep)

    @classmethod
    def load_device(cls, path, n_rows, n_cols, nnz, d_row_ptr, d_col_ind, K, options=None, keep=None):
        h = c_void_p()
        check(lib().sddmm_plan_load_device(str(path).encode(), n_rows, n_cols, nnz, c_void_p(d_row_ptr), c_void_p(d_col_ind), K,
                                           byref(options) if options is not None else None, byref(h)))
        return cls(h, keep)

    def save(self, path):
        check(lib().sddmm_plan_save(self.h, str(path).encode()))

    def options(self):
        o = PlanOptions()
        check(lib().sddmm_plan_get_options(self.h, byref(o)))
        return o.as_dict()

    def set_values(self, d_val, stream=0):
        check(lib().sddmm_plan_set_values(self.h, c_void_p(d_val), c_void_p(stream or None)))

    def info(self):
        i = PlanInfo()
        check(lib().sddmm_plan_get_info(self.h, byref(i)))
        return i.as_dict()

    def execute(self, d_val, d_W, d_H, d_out, stream=0):
        check(lib().sddmm_execute(self.h, c_void_p(d_val or None), c_void_p(d_W), c_void_p(d_H), c_void_p(d_out),
                                  c_void_p(stream or None)))

    def execute_epilogue(self, d_val, d_W, d_H, d_out, epilogue, stream=0):
        check(lib().sddmm_execute_epilogue(self.h, c_void_p(d_val or None), c_void_p(d_W), c_void_p(d_H), c_void_p(d_out),
                                           c_int32(epilogue), c_void_p(stream or None)))

    def execute_softmax(self, d_val, d_W, d_H, d_out, stream=0):
        check(lib().sddmm_execute_softmax(self.h, c_void_p(d_val or None), c_void_p(d_W), c_void_p(d_H), c_void_p(d_out),
                                          c_void_p(stream or None)))

    def workspace_bytes(self):
        n = c_int64()
        check(lib().sddmm_plan_workspace_bytes(self.h, byref(n)))
        return n.value

    def execute_ws(self, d_val, d_W, d_H, d_out, d_workspace, workspace_bytes, form=0, stream=0):
        """sddmm_execute_ws: form = EPILOGUE_SCALE / EPILOGUE_RESIDUAL, ored with FORM_SOFTMAX."""
        check(lib().sddmm_execute_ws(self.h, c_void_p(d_val or None), c_void_p(d_W), c_void_p(d_H), c_void_p(d_out), c_int32(form),
                                     c_void_p(d_workspace or None), c_int64(workspace_bytes), c_void_p(stream or None)))

    def spmm(self, d_x, d_H, d_Y, d_workspace=0, workspace_bytes=0, stream=0):
        check(lib().sddmm_plan_spmm(self.h, c_void_p(d_x or None), c_void_p(d_H), c_void_p(d_Y), c_void_p(d_workspace or None),
                                    c_int64(workspace_bytes), c_void_p(stream or None)))

    def execute_profiled(self, d_val, d_W, d_H, d_out, stream=0):
        n = c_int32()
        check(lib().sddmm_plan_launch_count(self.h, byref(n)))
        prof = (LaunchProfile * max(n.value, 1))()
        check(lib().sddmm_execute_profiled(self.h, c_void_p(d_val or None), c_void_p(d_W), c_void_p(d_H), c_void_p(d_out),
                                           c_void_p(stream or None), prof, n.value))
        return [{f: getattr(prof[i], f) for f, _ in LaunchProfile._fields_} for i in range(n.value)]

    def gpu(self, W, H):
        """Host arrays in, host array out (+ kernel-only ms): the calling
        convention of the reference's sddmm_GPU."""
        i = self.info()
        W = np.ascontiguousarray(W, np.float32)
        H = np.ascontiguousarray(H, np.float32)
        assert W.size == i["n_rows"] * i["K"] and H.size == i["n_cols"] * i["K"]
        out = np.empty(i["nnz"], np.float32)
        ms = c_float()
        check(lib().sddmm_gpu(self.h, _np_ptr(W), _np_ptr(H), _np_ptr(out), byref(ms)))
        return out, ms.value

    def close(self):
        if self.h:
            lib().sddmm_plan_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def init_reference(n, k):
    X = np.empty((n, k), np.float32)
    check(lib().sddmm_init_reference(_np_ptr(X), n, k))
    return X


def csr_noalloc(n_rows, n_cols, nnz, d_row_ptr, d_col_ind, d_val, K, d_W, d_H, d_out, stream=0):
    """Plan-free SDDMM over a device CSR that allocates nothing (sddmm_csr_noalloc)."""
    check(lib().sddmm_csr_noalloc(n_rows, n_cols, nnz, c_void_p(d_row_ptr), c_void_p(d_col_ind), c_void_p(d_val or None), K,
                                  c_void_p(d_W), c_void_p(d_H), c_void_p(d_out), c_void_p(stream or None)))


def row_softmax(n_rows, d_row_ptr, d_x, d_out, stream=0):
    check(lib().sddmm_row_softmax(n_rows, c_void_p(d_row_ptr), c_void_p(d_x), c_void_p(d_out), c_void_p(stream or None)))


def spmm_csr(n_rows, n_cols, nnz, d_row_ptr, d_col_ind, d_x, K, d_H, d_Y, stream=0):
    check(lib().sddmm_spmm_csr(n_rows, n_cols, nnz, c_void_p(d_row_ptr), c_void_p(d_col_ind or None), c_void_p(d_x or None), K,
                               c_void_p(d_H or None), c_void_p(d_Y), c_void_p(stream or None)))


def copy_probe(d_src, d_dst, n_bytes, stream=0):
    """Plain copy kernel of known size (sddmm_copy_probe), the reference HBM counters are scaled by."""
    check(lib().sddmm_copy_probe(c_void_p(d_src), c_void_p(d_dst), n_bytes, c_void_p(stream or None)))


def device_info():
    n = c_int()
    buf = C.create_string_buffer(256)
    lib().sddmm_device_info(byref(n), buf, 256)
    return n.value, buf.value.decode()
