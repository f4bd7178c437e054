// The planner of the SDDMM engine for gfx950 (MI355X): row classes, launch builders (row gather,
// unpadded LDS tiles, dense blocks, panels; the tile launch is in planner_tile.hip), options and
// their environment layer, kernel lookup, pattern hashes, workspace layout.
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstring>
#include <new>
#include <unistd.h>
#include "plan.hpp"

namespace sddmm {


// Batch side arrays for a stream whose segment s covers stream positions
// [seg_end[s-1], seg_end[s]) (seg_end increasing, last == stream length), for
// the batches of the given items.
void build_batches(const std::vector<WorkItem> &items, const int32_t *seg_end, int64_t n_seg,
                   std::vector<int32_t> &batch_seg, std::vector<uint64_t> &batch_mask)
{
    int64_t nb_total = 0;
    if (!items.empty()) {
        const WorkItem &last = items.back();
        nb_total = last.batch_base + ((int64_t)last.end - last.begin + 63) / 64;
    }
    batch_seg.assign((size_t)nb_total, 0);
    batch_mask.assign((size_t)nb_total, 0);
    auto fill = [&](const WorkItem &wi, int64_t b_lo, int64_t b_hi) {
        int64_t s = std::upper_bound(seg_end, seg_end + n_seg, (int32_t)(wi.begin + b_lo * 64)) - seg_end;
        for (int64_t b = b_lo; b < b_hi; ++b) {
            int64_t p0 = wi.begin + b * 64, p1 = std::min<int64_t>(p0 + 64, wi.end);
            while (s < n_seg && seg_end[s] <= p0) ++s;
            batch_seg[wi.batch_base + b] = (int32_t)s;
            uint64_t m = 0;
            int64_t t = s;
            while (t < n_seg && seg_end[t] < p1) {  // segment t+1 starts at seg_end[t], inside (p0, p1)
                if (seg_end[t] > p0) m |= 1ull << (seg_end[t] - p0);
                ++t;
            }
            batch_mask[wi.batch_base + b] = m;
        }
    };
    if (items.size() == 1) {  // one long item: split its batches over the threads
        const WorkItem &wi = items[0];
        int64_t nb = ((int64_t)wi.end - wi.begin + 63) / 64;
        parallel_ranges(nb, 1 << 12, [&](int64_t lo, int64_t hi, int) { fill(wi, lo, hi); });
        return;
    }
    parallel_ranges((int64_t)items.size(), 4, [&](int64_t ib, int64_t ie, int) {
        for (int64_t k = ib; k < ie; ++k) {
            const WorkItem &wi = items[k];
            if (wi.end > wi.begin) fill(wi, 0, ((int64_t)wi.end - wi.begin + 63) / 64);
        }
    });
}

int count_touched(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr, const int32_t *col_ind,
                  int64_t *rows_touched, int64_t *cols_touched)
{
    int64_t rt = 0;
    for (int64_t r = 0; r < n_rows; ++r) rt += row_ptr[r + 1] > row_ptr[r];
    std::vector<uint8_t> seen((size_t)n_cols, 0);
    parallel_ranges(nnz, 1 << 16, [&](int64_t b, int64_t e, int) {
        for (int64_t i = b; i < e; ++i) __atomic_store_n(&seen[col_ind[i]], (uint8_t)1, __ATOMIC_RELAXED);
    });
    int64_t ct = 0;
    for (int64_t c = 0; c < n_cols; ++c) ct += seen[c];
    *rows_touched = rt;
    *cols_touched = ct;
    return SDDMM_OK;
}

int device_ok()
{
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n < 1)
        return fail(SDDMM_ERR_HIP, "no HIP device available (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    return SDDMM_OK;
}

int64_t env_i64(const char *name, int64_t dflt)
{
    const char *e = getenv(name);
    if (!e || !*e) return dflt;
    char *end = nullptr;
    long long v = strtoll(e, &end, 10);
    return (end && *end == 0) ? (int64_t)v : dflt;
}

void default_options(sddmm_plan_options &o)
{
    memset(&o, 0, sizeof o);
    o.kernel = SDDMM_KERNEL_AUTO;
    o.tile_size_x = 0; o.tile_size_y = 0;
    o.k_slice = -1; o.tile_lanes = -1; o.tile_waves = -1; o.tile_assign = -1; o.tile_few_blocks = -1;
    o.tile_short_batches = -1; o.tile_deal = -1; o.tile_runs = -1; o.fuse_slices = -1; o.gather_lanes = -1; o.gather_padded = -1;
    o.gather_sink = -1; o.row_padded = -1; o.unpadded_tile = -1; o.dense_blocks = -1; o.dense_permille = -1;
    o.dense_rb_group = -1; o.ignore_env = 0;
    o.matrix_rows = -1; o.matrix_permille = -1; o.matrix_waves = -1; o.spmm_stream = -1;
    o.gather_slab_cols = -1; o.gather_panel_rows = -1; o.dense_min_nnz = -1; o.panel_bytes = -1; o.short_row_max = -1; o.stage_factor = -1; o.split_min_nnz = -1;
}

// The environment as an override layer over the caller's options.
void apply_env_overrides(sddmm_plan_options &o)
{
    if (o.ignore_env) return;
    auto i32 = [](const char *name, int32_t &v) { v = (int32_t)env_i64(name, v); };
    auto i64 = [](const char *name, int64_t &v) { v = env_i64(name, v); };
    i32("SDDMM_KERNEL", o.kernel); i32("SDDMM_TILE_X", o.tile_size_x); i32("SDDMM_TILE_Y", o.tile_size_y);
    i32("SDDMM_TILE_KSLICE", o.k_slice); i32("SDDMM_TILE_G", o.tile_lanes); i32("SDDMM_TILE_WAVES", o.tile_waves);
    i32("SDDMM_TILE_ASSIGN", o.tile_assign); i32("SDDMM_TILE_FEW_BLOCKS", o.tile_few_blocks);
    i32("SDDMM_TILE_SHORT", o.tile_short_batches); i32("SDDMM_TILE_DEAL", o.tile_deal); i32("SDDMM_TILE_RUNS", o.tile_runs); i32("SDDMM_FUSE_SLICES", o.fuse_slices);
    i32("SDDMM_GATHER_G", o.gather_lanes); i32("SDDMM_GATHER_PADDED", o.gather_padded); i32("SDDMM_GATHER_SINK", o.gather_sink);
    i32("SDDMM_ROW_PADDED", o.row_padded); i32("SDDMM_UNPADDED_TILE", o.unpadded_tile); i32("SDDMM_DENSE", o.dense_blocks);
    i32("SDDMM_DENSE_PERMILLE", o.dense_permille); i32("SDDMM_DENSE_RB_GROUP", o.dense_rb_group);
    i32("SDDMM_MATRIX_ROWS", o.matrix_rows); i32("SDDMM_MATRIX_PERMILLE", o.matrix_permille); i32("SDDMM_MATRIX_WAVES", o.matrix_waves);
    i32("SDDMM_SPMM_STREAM", o.spmm_stream);
    i64("SDDMM_GATHER_SLAB_COLS", o.gather_slab_cols); i64("SDDMM_GATHER_PANEL_ROWS", o.gather_panel_rows); i64("SDDMM_DENSE_MIN_NNZ", o.dense_min_nnz); i64("SDDMM_PANEL_BYTES", o.panel_bytes);
    i64("SDDMM_SHORT_ROW_MAX", o.short_row_max); i64("SDDMM_STAGE_FACTOR", o.stage_factor);
    i64("SDDMM_SPLIT_MIN_NNZ", o.split_min_nnz);
}

// Looks the launch's kernels up from its descriptor (fn_kind, fn_*, k_slice) and allows them its LDS size.
int resolve_functions(Launch &L)
{
    L.fn = nullptr; L.pfn = nullptr; L.tfn = nullptr; L.dfn = nullptr;
    for (auto &row : L.tfns) for (auto &f : row) f = nullptr;
    switch (L.fn_kind) {
    case 1:
    case 2: {
        const Variant v{L.fn_g, L.fn_kpl, L.fn_exact != 0};
        L.fn = v.G ? stream_kernel(v, L.fn_kind == 2) : (L.fn_kind == 1 ? generic_kernel() : nullptr);
        if (!L.fn) return fail(SDDMM_ERR_ARG, "plan: no stream kernel for lanes %d x %d", v.G, v.KPL);
        if (L.lds > 0) HIP_TRY(hipFuncSetAttribute((const void *)L.fn, hipFuncAttributeMaxDynamicSharedMemorySize, L.lds));
        return SDDMM_OK;
    }
    case 3: {
        const TileVariant tv{L.fn_g, L.fn_kpl};
        if (L.sp_on && spmm_tile_set_lds(L.k_slice, L.sp_nwaves, L.k_slice * 4 * L.ta.tile_x) != 0)
            return fail(SDDMM_ERR_HIP, "plan: cannot set up the tile kernel of the product Y = X H");
        if (L.fn_nwm > 0) {  // (a launch with a matrix-core share covers all of K: one form per value mode)
            for (int vm = 0; vm < 5; ++vm) {
                L.tfns[vm][0] = tile_kernel_mf(vm, L.fn_nwaves, L.fn_nwm);
                if (!L.tfns[vm][0]) return fail(SDDMM_ERR_ARG, "plan: no tile kernel with %d + %d waves", L.fn_nwaves, L.fn_nwm);
                HIP_TRY(hipFuncSetAttribute((const void *)L.tfns[vm][0], hipFuncAttributeMaxDynamicSharedMemorySize, L.lds));
            }
            L.fused_slices = 0;
            L.tfn = L.tfns[0][0];
            return SDDMM_OK;
        }
        for (int vm = 0; vm < 5; ++vm)
            for (int ac = 0; ac < 4; ++ac) {
                L.tfns[vm][ac] = tile_kernel(tv, vm, L.fn_gather != 0, ac, L.fn_nwaves);
                if (!L.tfns[vm][ac] && ac == 3) { L.fused_slices = 0; continue; }  // (that form exists for some variants only)
                if (!L.tfns[vm][ac]) return fail(SDDMM_ERR_ARG, "plan: no tile kernel for lanes %d x %d", tv.G, tv.KPL);
                HIP_TRY(hipFuncSetAttribute((const void *)L.tfns[vm][ac], hipFuncAttributeMaxDynamicSharedMemorySize, L.lds));
            }
        L.tfn = L.tfns[0][0];
        return SDDMM_OK;
    }
    case 4: {
        L.pfn = panel_kernel(pick_panel_variant(L.k_slice));
        if (!L.pfn) return fail(SDDMM_ERR_ARG, "plan: no panel kernel for K slice %d", L.k_slice);
        if (L.lds > 0) HIP_TRY(hipFuncSetAttribute((const void *)L.pfn, hipFuncAttributeMaxDynamicSharedMemorySize, L.lds));
        return SDDMM_OK;
    }
    case 5:
        L.dfn = dense_kernel();
        return SDDMM_OK;
    }
    return fail(SDDMM_ERR_FORMAT, "plan: unknown kernel descriptor %d", L.fn_kind);
}

// Order-independent 64-bit hash of a CSR pattern: the wrapping sum of a mixed word per row
// pointer and per column index (position included), so that the host (threads) and the device
// (atomic adds) arrive at the same value whatever order they visit the entries in.
__host__ __device__ inline uint64_t hash_row(int64_t r, int32_t v) { return mix64(((uint64_t)r << 32) ^ (uint32_t)v ^ 0x9e3779b97f4a7c15ull); }
__host__ __device__ inline uint64_t hash_col(int64_t i, int32_t v) { return mix64(((uint64_t)i << 32) | (uint32_t)v); }

uint64_t pattern_hash_host(int64_t n_rows, int64_t nnz, const int32_t *row_ptr, const int32_t *col_ind)
{
    std::vector<uint64_t> part((size_t)hw_threads() + 1, 0);
    parallel_ranges(n_rows + 1, 1 << 14, [&](int64_t b, int64_t e, int t) {
        uint64_t h = 0;
        for (int64_t r = b; r < e; ++r) h += hash_row(r, row_ptr[r]);
        part[(size_t)t] += h;
    });
    uint64_t h0 = 0;
    for (auto &x : part) { h0 += x; x = 0; }
    parallel_ranges(nnz, 1 << 16, [&](int64_t b, int64_t e, int t) {
        uint64_t h = 0;
        for (int64_t i = b; i < e; ++i) h += hash_col(i, col_ind[i]);
        part[(size_t)t] += h;
    });
    for (uint64_t x : part) h0 += x;
    return h0;
}

__global__ void pattern_hash_kernel(const int32_t *row_ptr, int64_t n_rows1, const int32_t *col_ind, int64_t nnz,
                                    unsigned long long *acc)
{
    uint64_t h = 0;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x, t0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (int64_t r = t0; r < n_rows1; r += stride) h += hash_row(r, row_ptr[r]);
    for (int64_t i = t0; i < nnz; i += stride) h += hash_col(i, col_ind[i]);
    // one atomic per wave: the lanes' sums are added up first
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t lo = __shfl_xor((uint32_t)h, off), hi = __shfl_xor((uint32_t)(h >> 32), off);
        h += ((uint64_t)hi << 32) | lo;
    }
    if ((threadIdx.x & 63) == 0) atomicAdd(acc, (unsigned long long)h);
}

int pattern_hash_device(int64_t n_rows, int64_t nnz, const int32_t *d_row_ptr, const int32_t *d_col_ind, uint64_t *out)
{
    unsigned long long *d_acc = nullptr;
    HIP_TRY(hipMalloc((void **)&d_acc, 8));
    struct Free { void *p; ~Free() { (void)hipFree(p); } } fr{d_acc};
    HIP_TRY(hipMemset(d_acc, 0, 8));
    hipLaunchKernelGGL(pattern_hash_kernel, dim3(2048), dim3(256), 0, nullptr, d_row_ptr, n_rows + 1, d_col_ind, nnz, d_acc);
    HIP_TRY(hipGetLastError());
    unsigned long long h = 0;
    HIP_TRY(hipMemcpy(&h, d_acc, 8, hipMemcpyDeviceToHost));
    *out = (uint64_t)h;
    return SDDMM_OK;
}

int64_t list_nnz(const Ctx &c, const std::vector<int32_t> &rows)
{
    int64_t n = 0;
    for (int32_t r : rows) n += c.row_ptr[r + 1] - c.row_ptr[r];
    return n;
}

// Row-gather launch over the given non-empty rows (ascending).  all_rows: the
// list is every non-empty row of S, so the stream is S itself.
int add_row_gather(Ctx &c, const std::vector<int32_t> &rows, bool all_rows)
{
    Launch L;
    L.kind = SDDMM_KERNEL_ROW_GATHER;
    L.rows = (int64_t)rows.size();
    if (c.orig) all_rows = false;  // positions of the remainder are not positions of S
    const int64_t n = all_rows ? c.nnz : list_nnz(c, rows);
    L.nnz = n;
    if (n == 0) return SDDMM_OK;
    const bool vec4 = c.K % 4 == 0;
    Variant var = vec4 ? pick_variant(c.K, false) : Variant{0, 0, false};
    L.fn_kind = 1; L.fn_g = var.G; L.fn_kpl = var.KPL; L.fn_exact = var.exact;
    if (int rc = resolve_functions(L)) return rc;
    std::vector<int32_t> seg_end(rows.size()), perm;
    int64_t acc = 0;
    for (size_t i = 0; i < rows.size(); ++i) {
        acc += c.row_ptr[rows[i] + 1] - c.row_ptr[rows[i]];
        seg_end[i] = (int32_t)acc;
    }
    if (!all_rows) {
        perm.resize((size_t)n);
        parallel_ranges((int64_t)rows.size(), 1 << 10, [&](int64_t b, int64_t e, int) {
            for (int64_t i = b; i < e; ++i) {
                int64_t d = i ? seg_end[i - 1] : 0;
                for (int32_t p = c.row_ptr[rows[i]]; p < c.row_ptr[rows[i] + 1]; ++p) perm[d++] = c.pos(p);
            }
        });
    }
    std::vector<int32_t> batch_seg;
    std::vector<uint64_t> batch_mask;
    std::vector<WorkItem> one{{0, (int32_t)n, 0, -1}};  // batches are multiples of 64 from 0
    build_batches(one, seg_end.data(), (int64_t)seg_end.size(), batch_seg, batch_mask);
    KArgs &a = L.ka;
    int32_t *d_seg_row = nullptr, *d_perm = nullptr, *d_bseg = nullptr;
    uint64_t *d_bmask = nullptr;
    if (!(all_rows && (int64_t)rows.size() == c.n_rows))
        if (int rc = c.up(&d_seg_row, rows)) return rc;
    if (int rc = c.up(&d_perm, perm)) return rc;
    if (int rc = c.up(&d_bseg, batch_seg)) return rc;
    if (int rc = c.up(&d_bmask, batch_mask)) return rc;
    a.seg_row = d_seg_row; a.perm = d_perm; a.batch_seg = d_bseg; a.batch_mask = d_bmask;
    L.perm = d_perm;
    a.nnz = (int32_t)n;
    // nonzeros per workgroup: up to 8 batches of 64 per wave, fewer when that would leave compute units idle
    const int64_t waves_wanted = 2 * (int64_t)c.cus * (kRowGatherBlock / 64);
    const int per_wave = (int)std::clamp<int64_t>(n / (64 * waves_wanted), 1, kRowGatherBatchesPerWave);
    a.chunk = 64 * per_wave * (kRowGatherBlock / 64);
    a.K = c.K; a.n_cols = (int32_t)c.n_cols; a.tile_x = (int32_t)c.n_cols;
    a.generic_perm = var.G == 0;
    L.grid = (int32_t)((n + a.chunk - 1) / a.chunk);
    L.block = kRowGatherBlock;
    L.k_slice = c.K;
    c.P->info.lanes_per_nnz = var.G ? var.G : 8;
    L.gather_g = var.G ? var.G : 8; L.positions = n;
    c.P->launches.push_back(L);
    return SDDMM_OK;
}

// LDS-tile launch: the rows' nonzeros in tile order (tiles of x columns).
int add_lds_tile(Ctx &c, const std::vector<int32_t> &rows, bool all_rows, int32_t x, int32_t y, sddmm_plan_info *I)
{
    Launch L;
    L.kind = SDDMM_KERNEL_LDS_TILE;
    L.rows = (int64_t)rows.size();
    Variant var = pick_variant(c.K, true);
    if (!var.G) return fail(SDDMM_ERR_ARG, "plan: no LDS-tile kernel for K = %d", c.K);
    L.fn_kind = 2; L.fn_g = var.G; L.fn_kpl = var.KPL; L.fn_exact = var.exact;
    sddmm_tiling T;
    if (int rc = build_tiling(c.n_rows, c.n_cols, c.nnz, c.row_ptr, c.col_ind, x, y, T, all_rows ? nullptr : rows.data(),
                              (int64_t)rows.size()))
        return rc;
    const int64_t n = T.nnz;
    L.nnz = n;
    if (n == 0) return SDDMM_OK;
    // work items: row panels, cut further so that no item exceeds max_item nonzeros
    const int64_t max_item = std::max<int64_t>(64 * 16 * 4, 8 * (int64_t)x);
    std::vector<WorkItem> items;
    int64_t nbatch = 0, n_blocks = 0;
    for (int32_t j = 0; j < T.n_tiles; ++j) {
        int64_t begin = T.tile_ptr[j];
        for (int64_t b = T.block_ptr[j]; b < T.block_ptr[j + 1]; ++b) {
            int64_t end = T.block_end[b];
            ++n_blocks;
            int64_t parts = std::max<int64_t>(1, (end - begin + max_item - 1) / max_item);
            int64_t per = (((end - begin + parts - 1) / parts) + 63) / 64 * 64;
            for (int64_t s = begin; s < end; s += per) {
                int64_t e = std::min(end, s + per);
                items.push_back({(int32_t)s, (int32_t)e, (int32_t)nbatch, j});
                nbatch += (e - s + 63) / 64;
            }
            begin = end;
        }
    }
    std::vector<int32_t> batch_seg;
    std::vector<uint64_t> batch_mask;
    build_batches(items, T.active_end.data(), (int64_t)T.active_end.size(), batch_seg, batch_mask);
    // column indices (and the plan's own values) once more in tile order: coalesced reads
    std::vector<int32_t> scol((size_t)n);
    parallel_ranges(n, 1 << 16, [&](int64_t b, int64_t e, int) {
        for (int64_t i = b; i < e; ++i) scol[i] = c.col_ind[T.tiled_ind[i]];
    });
    std::vector<float> sval;
    if (c.vals) {
        sval.resize((size_t)n);
        parallel_ranges(n, 1 << 16, [&](int64_t b, int64_t e, int) {
            for (int64_t i = b; i < e; ++i) sval[i] = c.value(T.tiled_ind[i]);
        });
    }
    if (c.orig)
        parallel_ranges(n, 1 << 16, [&](int64_t b, int64_t e, int) {
            for (int64_t i = b; i < e; ++i) T.tiled_ind[i] = c.orig[T.tiled_ind[i]];
        });
    KArgs &a = L.ka;
    int32_t *d_perm = nullptr, *d_seg_row = nullptr, *d_bseg = nullptr, *d_scol = nullptr;
    uint64_t *d_bmask = nullptr;
    WorkItem *d_items = nullptr;
    float *d_sval = nullptr;
    if (int rc = c.up(&d_perm, T.tiled_ind)) return rc;
    if (int rc = c.up(&d_seg_row, T.active_row)) return rc;
    if (int rc = c.up(&d_items, items)) return rc;
    if (int rc = c.up(&d_bseg, batch_seg)) return rc;
    if (int rc = c.up(&d_bmask, batch_mask)) return rc;
    if (int rc = c.up(&d_scol, scol)) return rc;
    if (int rc = c.up(&d_sval, sval)) return rc;
    a.perm = d_perm; a.seg_row = d_seg_row; a.items = d_items; a.batch_seg = d_bseg; a.batch_mask = d_bmask;
    a.scol = d_scol;
    L.sval = d_sval; L.perm = d_perm; L.positions = n;
    a.n_items = (int32_t)items.size();
    a.nnz = (int32_t)n; a.K = c.K; a.tile_x = x; a.n_cols = (int32_t)c.n_cols;
    L.grid = (int32_t)std::max<int64_t>(1, std::min<int64_t>((int64_t)c.cus, (int64_t)items.size()));
    L.block = kLdsBlock;
    L.lds = (int32_t)((int64_t)x * c.K * 4);
    L.k_slice = c.K;
    if (int rc = resolve_functions(L)) return rc;
    if (I) {
        I->tile_size_x = x; I->tile_size_y = y; I->n_col_tiles = T.n_tiles;
        I->n_row_panels = (int32_t)((T.max_active_rows + y - 1) / y);
        I->n_blocks = n_blocks; I->lanes_per_nnz = var.G; I->lds_bytes = L.lds; I->grid = L.grid; I->block = L.block;
    }
    c.P->launches.push_back(L);
    return SDDMM_OK;
}

// Dense-block launch: the blocks found by find_dense_blocks, one workgroup per block at a time.
int add_dense(Ctx &c, const DenseBlocks &D, const float *vals_all)
{
    Launch L;
    L.kind = SDDMM_KERNEL_DENSE_BLOCK;
    L.fn_kind = 5;
    if (int rc = resolve_functions(L)) return rc;
    L.nnz = D.n_dense;
    const int64_t n_tiles = (int64_t)D.tile_rb.size();
    // Schedule: workgroup b runs on die b % 8 (each die has its own L2) and takes slots b, b + grid, ...
    // The blocks are ordered by (group of 8 row blocks, column group, row block) and cut into 8
    // consecutive parts, one per die: the workgroups of a die then work on a few row blocks times a
    // few neighbouring column groups at a time, so the W rows of those row blocks stay in that L2
    // for the whole sweep over the columns and an H row is fetched once for the 8 row blocks that
    // use it (row blocks of similar length have about the same dense columns).
    const int rb_group = (int)std::max<int64_t>(1, (c.opt.dense_rb_group > 0 ? c.opt.dense_rb_group : 8));
    std::vector<int32_t> order((size_t)n_tiles), cg((size_t)n_tiles);
    for (int64_t k = 0; k < n_tiles; ++k) {
        order[(size_t)k] = (int32_t)k;
        cg[(size_t)k] = (k > 0 && D.tile_rb[(size_t)k] == D.tile_rb[(size_t)k - 1]) ? cg[(size_t)k - 1] + 1 : 0;
    }
    std::sort(order.begin(), order.end(), [&](int32_t x, int32_t y) {
        const int32_t gx = D.tile_rb[(size_t)x] / rb_group, gy = D.tile_rb[(size_t)y] / rb_group;
        if (gx != gy) return gx < gy;
        if (cg[(size_t)x] != cg[(size_t)y]) return cg[(size_t)x] < cg[(size_t)y];
        return x < y;
    });
    const int grid = (int)std::max<int64_t>(8, std::min<int64_t>(2 * (int64_t)c.cus, (n_tiles + 7) / 8 * 8)) / 8 * 8;
    const int per_die = grid / 8;
    const int64_t part = (n_tiles + 7) / 8;
    const int64_t turns = (part + per_die - 1) / per_die;
    const int64_t n_slots = turns * grid;
    const int T = D.tile;
    std::vector<int32_t> slot_rows((size_t)(n_slots * T), 0), slot_cols((size_t)(n_slots * T), 0);
    std::vector<int2> slot_range((size_t)n_slots, make_int2(0, 0));
    for (int die = 0; die < 8; ++die)
        for (int64_t j = 0; j < part; ++j) {
            if (die * part + j >= n_tiles) break;
            const int64_t tile = order[(size_t)(die * part + j)];
            const int64_t slot = (j / per_die) * grid + (j % per_die) * 8 + die;
            std::copy(D.row_ids.begin() + (size_t)D.tile_rb[(size_t)tile] * T, D.row_ids.begin() + ((size_t)D.tile_rb[(size_t)tile] + 1) * T,
                      slot_rows.begin() + (size_t)(slot * T));
            std::copy(D.col_ids.begin() + (size_t)tile * T, D.col_ids.begin() + ((size_t)tile + 1) * T, slot_cols.begin() + (size_t)(slot * T));
            slot_range[(size_t)slot] = make_int2(D.tile_ptr[(size_t)tile], D.tile_ptr[(size_t)tile + 1]);
        }
    std::vector<float> nz_val;
    if (vals_all) {
        nz_val.resize((size_t)D.n_dense);
        parallel_ranges(D.n_dense, 1 << 16, [&](int64_t b, int64_t e, int) {
            for (int64_t i = b; i < e; ++i) nz_val[(size_t)i] = vals_all[D.nz_p[(size_t)i]];
        });
    }
    int32_t *d_rows = nullptr, *d_cols = nullptr, *d_p = nullptr;
    int2 *d_range = nullptr;
    uint16_t *d_rc = nullptr;
    float *d_v = nullptr;
    if (int rc = c.up(&d_rows, slot_rows)) return rc;
    if (int rc = c.up(&d_cols, slot_cols)) return rc;
    if (int rc = c.up(&d_range, slot_range)) return rc;
    if (int rc = c.up(&d_p, D.nz_p)) return rc;
    if (int rc = c.up(&d_rc, D.nz_rc)) return rc;
    if (int rc = c.up(&d_v, nz_val)) return rc;
    DenseArgs &a = L.da;
    a.slot_rows = d_rows; a.slot_cols = d_cols; a.slot_range = d_range;
    a.nz_p = d_p; a.nz_rc = d_rc;
    a.n_slots = (int32_t)n_slots; a.K = c.K;
    L.sval = d_v; L.perm = d_p; L.positions = D.n_dense;
    L.grid = grid; L.block = 256; L.lds = 0; L.k_slice = c.K;
    L.rows = (int64_t)D.row_ids.size();
    c.P->info.dense_nnz = D.n_dense;
    c.P->info.dense_blocks = n_tiles;
    c.P->launches.push_back(L);
    return SDDMM_OK;
}

// Panel launch over the given non-empty rows (ascending): K slices of ks.
int add_panel(Ctx &c, const std::vector<int32_t> &rows, int ks, int32_t tile_x, int32_t tile_y, sddmm_plan_info *I)
{
    Launch L;
    L.kind = SDDMM_KERNEL_PANEL;
    L.rows = (int64_t)rows.size();
    L.nnz = list_nnz(c, rows);
    if (L.nnz == 0) return SDDMM_OK;
    const PanelVariant pv = pick_panel_variant(ks);
    if (!panel_kernel(pv)) return fail(SDDMM_ERR_ARG, "plan: no panel kernel for K slice %d", ks);
    L.fn_kind = 4;
    const int32_t fit = kLdsMaxBytes / (ks * 4);
    int32_t x = tile_x > 0 ? std::min(tile_x, fit) : fit;
    x = (int32_t)std::min<int64_t>(x, std::max<int64_t>(c.n_cols, 1));
    const int octs_cap = pv.S * pv.NWAVES;  // octets (8 rows, one per lane group of a wave) per panel
    int octs = octs_cap;
    if (tile_y > 0) octs = (int)std::max<int64_t>(1, std::min<int64_t>(octs_cap, ((int64_t)tile_y + 7) / 8));
    // spread a small row set over the CUs rather than filling few panels to the brim
    {
        int64_t want_panels = std::min<int64_t>(c.cus, ((int64_t)rows.size() + 63) / 64);
        int64_t octs_even = (((int64_t)rows.size() + want_panels - 1) / want_panels + 7) / 8;
        if (tile_y <= 0) octs = (int)std::max<int64_t>(1, std::min<int64_t>(octs, octs_even));
    }
    const int rows_per_panel = octs * 8;
    // panels: contiguous runs of the rows (keeps the column locality of neighbouring
    // rows); inside a panel rows are ranked by length so that the 8 groups of a
    // wave work on rows of similar length in the same slot
    const int64_t n_panels = ((int64_t)rows.size() + rows_per_panel - 1) / rows_per_panel;
    std::vector<int32_t> slot_row((size_t)n_panels * pv.S * pv.NWAVES * 8, -1);
    std::vector<int32_t> panel_tiles((size_t)n_panels * 2, 0);
    const int32_t *row_ptr = c.row_ptr, *col_ind = c.col_ind;
    parallel_ranges(n_panels, 4, [&](int64_t pb, int64_t pe, int) {
        std::vector<int32_t> rk;
        for (int64_t p = pb; p < pe; ++p) {
            const int64_t b = p * rows_per_panel, e = std::min<int64_t>(b + rows_per_panel, (int64_t)rows.size());
            rk.assign(rows.begin() + b, rows.begin() + e);
            std::stable_sort(rk.begin(), rk.end(), [&](int32_t u, int32_t v) {
                return row_ptr[u + 1] - row_ptr[u] > row_ptr[v + 1] - row_ptr[v];
            });
            int32_t cmin = INT32_MAX, cmax = 0;
            for (size_t i = 0; i < rk.size(); ++i) {
                const int oct = (int)(i / 8), g = (int)(i % 8);
                const int slot = oct / pv.NWAVES, wave = oct % pv.NWAVES;
                slot_row[((((size_t)p * pv.S + slot) * pv.NWAVES) + wave) * 8 + g] = rk[i];
                cmin = std::min(cmin, col_ind[row_ptr[rk[i]]]);
                cmax = std::max(cmax, col_ind[row_ptr[rk[i] + 1] - 1]);
            }
            panel_tiles[2 * p] = cmin / x;
            panel_tiles[2 * p + 1] = cmax / x;
        }
    });
    if (int rc = c.need_row_ptr()) return rc;
    int32_t *d_slot = nullptr, *d_pt = nullptr;
    if (int rc = c.up(&d_slot, slot_row)) return rc;
    if (int rc = c.up(&d_pt, panel_tiles)) return rc;
    PanelArgs &pa = L.pa;
    pa.slot_row = d_slot; pa.panel_tiles = d_pt;
    pa.n_panels = (int32_t)n_panels; pa.tile_x = x; pa.n_cols = (int32_t)c.n_cols; pa.K = c.K;
    L.grid = (int32_t)std::max<int64_t>(1, std::min<int64_t>(c.cus, n_panels));
    L.block = pv.NWAVES * 64;
    L.lds = x * ks * 4;
    L.k_slice = ks;
    if (int rc = resolve_functions(L)) return rc;
    if (I) {
        I->tile_size_x = x; I->tile_size_y = rows_per_panel; I->k_slice = ks;
        I->n_col_tiles = (int32_t)((c.n_cols + x - 1) / x); I->n_row_panels = (int32_t)n_panels;
        I->n_blocks = 0;
        for (int64_t p = 0; p < n_panels; ++p) I->n_blocks += panel_tiles[2 * p + 1] - panel_tiles[2 * p] + 1;
        I->lanes_per_nnz = 8; I->grid = L.grid; I->block = L.block; I->lds_bytes = L.lds;
    }
    c.P->launches.push_back(L);
    return SDDMM_OK;
}

// Lays the scratch memory of every launch, and the records of the softmax pass, out in one block a caller can
// bring along (sddmm_execute_ws), each piece on a 256-byte boundary.
void assign_workspace(sddmm_plan *P)
{
    int64_t at = 0;
    auto take = [&](int64_t bytes) { const int64_t o = at; at += (bytes + 255) / 256 * 256; return o; };
    for (Launch &L : P->launches) {
        L.ws_part = take(L.part_bytes);
        L.ws_hp = take(L.hp_bytes);
        L.ws_wp = take(L.wp_bytes);
        L.ws_sp_part = take(L.sp_part_bytes);
    }
    P->ws_softmax = take(row_softmax_workspace_bytes(P->info.nnz));
    P->ws_bytes = at;
}

// Common plan builder from host CSR arrays.  d_*_borrowed != null: the device
// already holds that array.
int make_plan(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr_all, const int32_t *col_ind_all,
              const float *vals, const int32_t *d_row_ptr_borrowed, const int32_t *d_col_borrowed, int32_t K,
              const sddmm_plan_options &opt_in, sddmm_plan **out)
{
    sddmm_plan_options opt = opt_in;
    apply_env_overrides(opt);
    if (opt.tile_lanes < 0) opt.tile_lanes = 0;  // (0 is "choose" for the variant pickers)
    const int32_t tile_x = opt.tile_size_x, tile_y = opt.tile_size_y;
    auto t0 = std::chrono::steady_clock::now();
    if (K < 1) return fail(SDDMM_ERR_ARG, "plan: K must be >= 1 (got %d)", K);
    if (tile_x < 0 || tile_y < 0) return fail(SDDMM_ERR_ARG, "plan: tile sizes must be >= 0");
    if (nnz >= INT32_MAX - 4096 || n_rows >= INT32_MAX || n_cols >= INT32_MAX)
        return fail(SDDMM_ERR_RANGE, "plan: sizes beyond int32 offsets");
    if ((n_rows * (int64_t)K) >= (int64_t)1 << 40 || (n_cols * (int64_t)K) >= (int64_t)1 << 40)
        return fail(SDDMM_ERR_RANGE, "plan: dense factor too large");
    if (int rc = device_ok()) return rc;
    int want = opt.kernel;
    if (want < 0) return fail(SDDMM_ERR_ARG, "plan: unknown kernel id %d", want);
    if (want > SDDMM_KERNEL_HYBRID) return fail(SDDMM_ERR_ARG, "plan: unknown kernel id %d", want);

    sddmm_plan *P = new (std::nothrow) sddmm_plan;
    if (!P) return fail(SDDMM_ERR_NOMEM, "plan: out of memory");
    struct Guard { sddmm_plan *p; ~Guard() { delete p; } } guard{P};
    sddmm_plan_info &I = P->info;
    I.n_rows = n_rows; I.n_cols = n_cols; I.nnz = nnz; I.K = K; I.k_slice = K;
    count_touched(n_rows, n_cols, nnz, row_ptr_all, col_ind_all, &I.rows_touched, &I.cols_touched);
    P->requested_kernel = want;
    P->pattern_hash = pattern_hash_host(n_rows, nnz, row_ptr_all, col_ind_all);
    // what the gathering kernels work on: S itself, or what is left of it once the dense blocks are cut out
    const int32_t *row_ptr = row_ptr_all, *col_ind = col_ind_all;
    int64_t nnz_part = nnz;

    hipDeviceProp_t prop;
    int device = 0;
    HIP_TRY(hipGetDevice(&device));
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    Ctx c{P, n_rows, n_cols, nnz, row_ptr_all, col_ind_all, vals, K, prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256};
    c.opt = opt;
    P->options = opt;

    P->d_row_ptr = d_row_ptr_borrowed;
    if (d_col_borrowed) {
        P->d_col = d_col_borrowed;
    } else if (nnz) {
        int32_t *d = nullptr;
        HIP_TRY(hipMalloc((void **)&d, (size_t)nnz * 4));
        P->owned.push_back({d, (size_t)nnz * 4});
        HIP_TRY(hipMemcpy(d, col_ind_all, (size_t)nnz * 4, hipMemcpyHostToDevice));
        c.dev_bytes += nnz * 4;
        P->d_col = d;
    }
    if (vals && nnz) {
        HIP_TRY(hipMalloc((void **)&P->d_val, (size_t)nnz * 4));
        P->owned.push_back({P->d_val, (size_t)nnz * 4});
        HIP_TRY(hipMemcpy(P->d_val, vals, (size_t)nnz * 4, hipMemcpyHostToDevice));
        c.dev_bytes += nnz * 4;
    }

    const bool have_vec = (K % 4 == 0) && pick_variant(K, true).G != 0;
    const int64_t row_bytes = (int64_t)K * 4;
    const int32_t fit_x = (int32_t)std::min<int64_t>(kLdsMaxBytes / row_bytes, INT32_MAX);  // H rows per LDS tile at full K
    const int ks = (K % 128 == 0) ? 128 : (K % 64 == 0) ? 64 : (K % 32 == 0) ? 32 : 0;    // panel kernel K slice
    // K elements per launch of the tile kernel: all of K while a row of 128 floats or
    // less keeps tiles wide; beyond that, slices of 128 (or 64) accumulated into out
    int kt = 0;
    if (K <= 128 && pick_tile_variant(K, 0).G) kt = K;
    else if (K > 128 && K % 128 == 0) kt = 128;
    else if (K > 128 && K % 64 == 0) kt = 64;
    else if (pick_tile_variant(K, 0).G) kt = K;
    if (opt.k_slice > 0 && K % opt.k_slice == 0 && pick_tile_variant(opt.k_slice, 0).G) kt = opt.k_slice;
    const int32_t fit_t = kt ? kLdsMaxBytes / (kt * 4) : 0;  // H rows per LDS tile of the tile kernel

    // row-panel height of the tile kernel's stream: the panel's W slice (y rows of kt floats)
    // should stay L2-resident while the workgroups sweep the panel's column tiles
    int32_t y_panel = tile_y > 0 ? tile_y : (kt ? (int32_t)std::max<int64_t>(256, (opt.panel_bytes > 0 ? opt.panel_bytes : (int64_t)(2 << 20)) / (kt * 4)) : 1);

    int kernel = want;
    if (kernel == SDDMM_KERNEL_AUTO) kernel = SDDMM_KERNEL_HYBRID;
    if (kernel == SDDMM_KERNEL_LDS_TILE && !kt && (!have_vec || fit_x < 1)) kernel = SDDMM_KERNEL_ROW_GATHER;
    if (kernel == SDDMM_KERNEL_PANEL && ks == 0) kernel = SDDMM_KERNEL_ROW_GATHER;
    if (kernel == SDDMM_KERNEL_HYBRID && !kt) kernel = SDDMM_KERNEL_ROW_GATHER;

    I.tile_size_x = (int32_t)std::min<int64_t>(n_cols, INT32_MAX);
    I.tile_size_y = (int32_t)std::min<int64_t>(n_rows, INT32_MAX);
    I.n_col_tiles = 1; I.n_row_panels = 1; I.n_blocks = 1; I.lanes_per_nnz = 8;

    // The dense core first (HYBRID only, ranks the dense kernel's chunks divide, and only next to
    // the non-compact tile streams, which can address a remainder): blocks of 128 ranked rows x
    // 128 ranked columns filled to the threshold go to the matrix cores.
    DenseBlocks D;
    // Measured on the recommender shape it pays from K = 512 on (the remainder's shorter runs cost the
    // tile kernel what the matrix cores save below that), so that is where "choose" turns it on.
    const bool want_dense = opt.dense_blocks > 0 || (opt.dense_blocks < 0 && K >= 512);
    if (kernel == SDDMM_KERNEL_HYBRID && want_dense && K % 32 == 0 && kt / 4 > 16 &&
        (int64_t)n_rows * (K / 4) <= (int64_t)UINT32_MAX && (int64_t)n_cols * (K / 4) <= (int64_t)UINT32_MAX) {
        const double threshold = (double)(opt.dense_permille > 0 ? opt.dense_permille : 300) / 1000.0;
        const int64_t min_dense = opt.dense_min_nnz >= 0 ? opt.dense_min_nnz : std::max<int64_t>(nnz / 50, 1 << 20);
        // (a host too short of memory for the search plans without dense blocks)
        try {
            if (int rc = find_dense_blocks(n_rows, n_cols, nnz, row_ptr_all, col_ind_all, kDenseTile, threshold, min_dense, D)) return rc;
        } catch (const std::bad_alloc &) {
            D = DenseBlocks{};
        }
        if (D.n_dense > 0) {
            if (int rc = add_dense(c, D, vals)) return rc;
            row_ptr = D.rem_row_ptr.data(); col_ind = D.rem_col.data(); nnz_part = nnz - D.n_dense;
            c.row_ptr = row_ptr; c.col_ind = col_ind; c.nnz = nnz_part; c.orig = D.rem_orig.data();
        }
    }

    // non-empty rows, ascending
    std::vector<int32_t> ne;
    ne.reserve((size_t)I.rows_touched);
    for (int64_t r = 0; r < n_rows; ++r)
        if (row_ptr[r + 1] > row_ptr[r]) ne.push_back((int32_t)r);

    if (kernel == SDDMM_KERNEL_HYBRID) {
        // Rows are split by length into classes:
        //   long   tile kernel with the default group size
        //   medium (only with SDDMM_MED_CLASS=1) tile kernel with groups of 4 lanes: less
        //          padding on short runs, but twice the W bytes per position through the
        //          load path, which is what binds it -- measured no faster than "long"
        //   short  padded gather: a row has so few nonzeros per column tile that padded
        //          runs would mostly be padding
        // How many tiles a row's nonzeros spread over is judged from the column span of
        // panels of consecutive rows, not from n_cols (a banded matrix spans few tiles).
        int32_t x = tile_x > 0 ? std::min(tile_x, fit_t) : fit_t;
        x = (int32_t)std::min<int64_t>(x, std::max<int64_t>(n_cols, 1));
        double span = (double)n_cols;
        if (!ne.empty()) {
            const size_t chunk = 512;
            double acc = 0; int64_t cnt = 0;
            for (size_t b = 0; b < ne.size(); b += chunk * 16) {  // every 16th chunk of 512 rows
                size_t e2 = std::min(ne.size(), b + chunk);
                int32_t cmin = INT32_MAX, cmax = 0;
                for (size_t i = b; i < e2; ++i) {
                    cmin = std::min(cmin, col_ind[row_ptr[ne[i]]]);
                    cmax = std::max(cmax, col_ind[row_ptr[ne[i] + 1] - 1]);
                }
                acc += (double)(cmax - cmin + 1); ++cnt;
            }
            span = acc / (double)cnt;
        }
        const double tiles = std::max(1.0, span / std::max(1, x));
        const int g_long = pick_tile_variant(kt, opt.tile_lanes).G ? pick_tile_variant(kt, opt.tile_lanes).G : pick_tile_variant(kt, 0).G;
        // rows with at least short_max nonzeros (2 per column tile with groups of 8 lanes) go to the tile kernel
        int64_t short_max = (int64_t)std::max(4.0, (g_long == 8 ? 2.0 : 1.0 * g_long) * tiles);
        if (opt.short_row_max >= 0) short_max = opt.short_row_max;
        std::vector<int32_t> rl, rs;
        int64_t nl = 0, nsh = 0;
        for (int32_t r : ne) {
            const int64_t d = row_ptr[r + 1] - row_ptr[r];
            if (d >= short_max) { rl.push_back(r); nl += d; }
            else { rs.push_back(r); nsh += d; }
        }
        // staging every H tile must be paid for by the nonzeros that use it
        const int64_t n_tiles_all = (n_cols + x - 1) / x;
        const int64_t stage_rows = std::max<int64_t>(n_tiles_all, c.cus) * x;
        if (nl < (opt.stage_factor >= 0 ? opt.stage_factor : 8) * stage_rows) {
            rs.insert(rs.end(), rl.begin(), rl.end());
            nsh += nl; nl = 0; rl.clear();
            std::sort(rs.begin(), rs.end());
        }
        // a small problem is one launch: splitting it only adds launch latency
        if (nl && nnz_part < (opt.split_min_nnz >= 0 ? opt.split_min_nnz : (int64_t)4 * 1000 * 1000)) {
            rl.insert(rl.end(), rs.begin(), rs.end());
            nl += nsh; nsh = 0; rs.clear();
            std::sort(rl.begin(), rl.end());
        }
        // a class too small to fill the machine joins the other
        if (!rl.empty() && !rs.empty() && nl * 50 < nnz_part) {
            rs.insert(rs.end(), rl.begin(), rl.end());
            nsh += nl; nl = 0; rl.clear();
            std::sort(rs.begin(), rs.end());
        }
        // (a handful of short rows -- the clipped rows at the corners of a band -- are not worth a launch
        // of their own: a single workgroup would walk them batch by batch at memory latency;
        // banded 2^20, K = 512: 711 nonzeros took 0.065 ms of a 4.14 ms step)
        if (!rl.empty() && !rs.empty() && opt.short_row_max < 0 && nsh * 2000 < nnz_part) {
            rl.insert(rl.end(), rs.begin(), rs.end());
            nl += nsh; nsh = 0; rs.clear();
            std::sort(rl.begin(), rl.end());
        }
        if (!rl.empty())
            if (int rc = add_tile(c, rl, x, y_panel, opt.tile_lanes, kt, &I, false, tile_x > 0)) return rc;
        if (!rs.empty()) {
            // short rows: the padded, pipelined kernel reading H from global memory when the
            // rows are short enough for padding to stay cheap; the plain row gather otherwise
            // An H far larger than the caches (every die's 4 MB of L2, 32 MB together) and no tiled class:
            // every gathered H row would cross the fabric (R-MAT 2^22, K=64: 41.8 GB per step for 4.5 GB of
            // algorithmic bytes, 8.27 ms).  The padded gather then walks S in column slabs whose H rows
            // come to 32 MB, with groups of 4 lanes (runs inside a slab are short): 26.3 GB, 4.96 ms.
            // Narrower slabs lose to the W rows re-read per (row, slab) run, wider ones to H misses.
            const bool huge_h = rl.empty() && D.n_dense == 0 && (int64_t)n_cols * K * 4 > ((int64_t)256 << 20);
            int gg = opt.gather_lanes > 0 ? opt.gather_lanes : 8;
            if (huge_h && opt.gather_lanes <= 0 && opt.gather_slab_cols != 0 && pick_tile_variant(kt, 4).G) gg = 4;
            const bool slabs = huge_h && opt.gather_slab_cols != 0 && opt.gather_padded != 0 && pick_tile_variant(kt, gg).G != 0;
            const bool padded = opt.gather_padded != 0 && pick_tile_variant(kt, gg).G != 0 && (!rl.empty() || D.n_dense > 0 || slabs);
            if (padded) {
                const int64_t keep = c.opt.gather_slab_cols;
                if (slabs && keep < 0) c.opt.gather_slab_cols = std::max<int64_t>(1024, ((int64_t)32 << 20) / ((int64_t)K * 4));
                const int rc = add_tile(c, rs, 0, 0, gg, kt, nullptr, true);
                c.opt.gather_slab_cols = keep;
                if (rc) return rc;
            } else if (int rc = add_row_gather(c, rs, rs.size() == ne.size())) return rc;
        }
        I.kernel = (P->launches.size() == 1 && !P->launches[0].dfn) ? P->launches[0].kind : SDDMM_KERNEL_HYBRID;
        I.class_nnz[0] = nl; I.class_nnz[1] = 0; I.class_nnz[2] = nsh;
        I.class_rows[0] = (int64_t)rl.size(); I.class_rows[1] = 0; I.class_rows[2] = (int64_t)rs.size();
    } else if (kernel == SDDMM_KERNEL_PANEL) {
        if (int rc = add_panel(c, ne, ks, tile_x, tile_y, &I)) return rc;
        I.kernel = kernel; I.class_nnz[1] = nnz; I.class_rows[1] = (int64_t)ne.size();
    } else if (kernel == SDDMM_KERNEL_LDS_TILE) {
        int32_t y = tile_y > 0 ? tile_y : (int32_t)std::min<int64_t>(std::max<int64_t>(n_rows, 1), INT32_MAX);
        if (kt && opt.unpadded_tile <= 0) {
            int32_t x = tile_x > 0 ? std::min(tile_x, fit_t) : fit_t;
            x = (int32_t)std::min<int64_t>(x, std::max<int64_t>(n_cols, 1));
            if (int rc = add_tile(c, ne, x, tile_y > 0 ? tile_y : y_panel, opt.tile_lanes, kt, &I, false, tile_x > 0)) return rc;
        } else {
            int32_t x = tile_x > 0 ? std::min(tile_x, fit_x) : fit_x;
            x = (int32_t)std::min<int64_t>(x, std::max<int64_t>(n_cols, 1));
            if (int rc = add_lds_tile(c, ne, true, x, y, &I)) return rc;
        }
        I.kernel = kernel; I.class_nnz[0] = nnz; I.class_rows[0] = (int64_t)ne.size();
    } else {
        const int gg = opt.gather_lanes > 0 ? opt.gather_lanes : 0;
        if (opt.row_padded > 0 && kt && pick_tile_variant(kt, gg).G != 0) {
            if (int rc = add_tile(c, ne, 0, 0, gg, kt, &I, true)) return rc;
        } else if (int rc = add_row_gather(c, ne, true)) return rc;
        I.kernel = SDDMM_KERNEL_ROW_GATHER; I.class_nnz[2] = nnz; I.class_rows[2] = (int64_t)ne.size();
    }
    // the row pointers stay with the plan (the row-wise softmax epilogue walks S row by row)
    c.row_ptr = row_ptr_all;
    if (nnz > 0)
        if (int rc = c.need_row_ptr()) return rc;
    if (!P->launches.empty() && I.grid == 0) { I.grid = P->launches[0].grid; I.block = P->launches[0].block; I.lds_bytes = P->launches[0].lds; }
    I.n_launches = 0;
    for (const Launch &L : P->launches) I.n_launches += (L.k_slice > 0 && L.k_slice < K && !L.fused_slices) ? K / L.k_slice : 1;
    I.device_bytes = c.dev_bytes;
    assign_workspace(P);
    I.plan_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    guard.p = nullptr;
    *out = P;
    return SDDMM_OK;
}

}  // namespace sddmm
