// Plan construction (stream descriptors for the kernels, upload) and launch
// of the SDDMM engine for gfx950 (MI355X).
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstring>
#include <new>
#include "internal.hpp"
#include "kernels.hpp"

using namespace sddmm;

namespace {

#define HIP_TRY(expr)                                                                               \
    do {                                                                                            \
        hipError_t e_ = (expr);                                                                     \
        if (e_ != hipSuccess)                                                                       \
            return fail(SDDMM_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
    } while (0)

template <class T>
int upload(T **dst, const std::vector<T> &src, int64_t *bytes)
{
    *dst = nullptr;
    if (src.empty()) return SDDMM_OK;
    HIP_TRY(hipMalloc((void **)dst, src.size() * sizeof(T)));
    HIP_TRY(hipMemcpy(*dst, src.data(), src.size() * sizeof(T), hipMemcpyHostToDevice));
    *bytes += (int64_t)(src.size() * sizeof(T));
    return SDDMM_OK;
}

}  // namespace

struct sddmm_plan {
    sddmm_plan_info info{};
    Variant variant{0, 0, false};
    KernelFn fn = nullptr;
    const int32_t *d_col = nullptr;
    bool own_col = false;
    float *d_val = nullptr;
    int32_t *d_perm = nullptr, *d_seg_row = nullptr, *d_batch_seg = nullptr;
    uint64_t *d_batch_mask = nullptr;
    WorkItem *d_items = nullptr;
    int32_t n_items = 0;
    int32_t chunk = 0;
    // panel kernel
    PanelFn panel_fn = nullptr;
    const int32_t *d_row_ptr = nullptr;
    bool own_row_ptr = false;
    int32_t *d_slot_row = nullptr, *d_panel_tiles = nullptr;
    int32_t n_panels = 0;
    ~sddmm_plan()
    {
        if (own_row_ptr && d_row_ptr) (void)hipFree((void *)d_row_ptr);
        if (d_slot_row) (void)hipFree(d_slot_row);
        if (d_panel_tiles) (void)hipFree(d_panel_tiles);
        if (own_col && d_col) (void)hipFree((void *)d_col);
        if (d_val) (void)hipFree(d_val);
        if (d_perm) (void)hipFree(d_perm);
        if (d_seg_row) (void)hipFree(d_seg_row);
        if (d_batch_seg) (void)hipFree(d_batch_seg);
        if (d_batch_mask) (void)hipFree(d_batch_mask);
        if (d_items) (void)hipFree(d_items);
    }
};

namespace {

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
    parallel_ranges((int64_t)items.size(), 4, [&](int64_t ib, int64_t ie, int) {
        for (int64_t k = ib; k < ie; ++k) {
            const WorkItem &wi = items[k];
            if (wi.end <= wi.begin) continue;
            int64_t s = std::upper_bound(seg_end, seg_end + n_seg, wi.begin) - seg_end;  // segment of wi.begin
            int64_t nb = ((int64_t)wi.end - wi.begin + 63) / 64;
            for (int64_t b = 0; b < nb; ++b) {
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

// Common plan builder from host CSR arrays.  d_col_borrowed != null: the
// device already holds col_ind.
int make_plan(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr, const int32_t *col_ind,
              const float *vals, const int32_t *d_row_ptr_borrowed, const int32_t *d_col_borrowed, int32_t K, int32_t tile_x, int32_t tile_y,
              uint32_t flags, sddmm_plan **out)
{
    auto t0 = std::chrono::steady_clock::now();
    if (K < 1) return fail(SDDMM_ERR_ARG, "plan: K must be >= 1 (got %d)", K);
    if (tile_x < 0 || tile_y < 0) return fail(SDDMM_ERR_ARG, "plan: tile sizes must be >= 0");
    if (nnz >= INT32_MAX - 4096 || n_rows >= INT32_MAX || n_cols >= INT32_MAX)
        return fail(SDDMM_ERR_RANGE, "plan: sizes beyond int32 offsets");
    if ((n_rows * (int64_t)K) >= (int64_t)1 << 40 || (n_cols * (int64_t)K) >= (int64_t)1 << 40)
        return fail(SDDMM_ERR_RANGE, "plan: dense factor too large");
    if (int rc = device_ok()) return rc;
    int want = (int)(flags & 0xff);
    if (want > SDDMM_KERNEL_PANEL) return fail(SDDMM_ERR_ARG, "plan: unknown kernel id %d", want);

    sddmm_plan *P = new (std::nothrow) sddmm_plan;
    if (!P) return fail(SDDMM_ERR_NOMEM, "plan: out of memory");
    struct Guard { sddmm_plan *p; ~Guard() { delete p; } } guard{P};
    sddmm_plan_info &I = P->info;
    I.n_rows = n_rows; I.n_cols = n_cols; I.nnz = nnz; I.K = K; I.k_slice = K;
    count_touched(n_rows, n_cols, nnz, row_ptr, col_ind, &I.rows_touched, &I.cols_touched);

    const bool vec4 = (K % 4 == 0);
    Variant var = vec4 ? pick_variant(K) : Variant{0, 0, false};
    const bool have_fast = var.G != 0;

    // kernel choice
    int kernel = want;
    const int64_t row_bytes = (int64_t)K * 4;
    int32_t fit_x = (int32_t)std::min<int64_t>(kLdsMaxBytes / row_bytes, INT32_MAX);
    if (kernel == SDDMM_KERNEL_AUTO)
        kernel = (have_fast && tile_x > 0 && tile_x < n_cols && fit_x >= 8) ? SDDMM_KERNEL_LDS_TILE : SDDMM_KERNEL_ROW_GATHER;
    if (kernel == SDDMM_KERNEL_LDS_TILE && (!have_fast || fit_x < 1)) kernel = SDDMM_KERNEL_ROW_GATHER;
    // the panel kernel works on K slices of 128, 64 or 32 elements
    const int ks = (K % 128 == 0) ? 128 : (K % 64 == 0) ? 64 : (K % 32 == 0) ? 32 : 0;
    if (kernel == SDDMM_KERNEL_PANEL && ks == 0) kernel = SDDMM_KERNEL_ROW_GATHER;
    I.kernel = kernel;
    I.lanes_per_nnz = have_fast ? var.G : 8;
    P->variant = var;

    int64_t dev_bytes = 0;
    if (d_col_borrowed) {
        P->d_col = d_col_borrowed;
    } else {
        int32_t *d = nullptr;
        if (nnz) {
            HIP_TRY(hipMalloc((void **)&d, (size_t)nnz * 4));
            HIP_TRY(hipMemcpy(d, col_ind, (size_t)nnz * 4, hipMemcpyHostToDevice));
            dev_bytes += nnz * 4;
        }
        P->d_col = d; P->own_col = true;
    }
    if (vals && nnz) {
        HIP_TRY(hipMalloc((void **)&P->d_val, (size_t)nnz * 4));
        HIP_TRY(hipMemcpy(P->d_val, vals, (size_t)nnz * 4, hipMemcpyHostToDevice));
        dev_bytes += nnz * 4;
    }

    std::vector<int32_t> batch_seg;
    std::vector<uint64_t> batch_mask;
    if (kernel == SDDMM_KERNEL_PANEL) {
        const PanelVariant pv = pick_panel_variant(ks);
        P->panel_fn = panel_kernel(pv);
        if (!P->panel_fn) return fail(SDDMM_ERR_ARG, "plan: no panel kernel for K slice %d", ks);
        const int32_t fit = kLdsMaxBytes / (ks * 4);
        int32_t x = tile_x > 0 ? std::min(tile_x, fit) : fit;
        x = (int32_t)std::min<int64_t>(x, std::max<int64_t>(n_cols, 1));
        const int octs_cap = pv.S * pv.NWAVES;  // octets (8 rows, one per lane group of a wave) per panel
        int octs = octs_cap;
        if (tile_y > 0) octs = (int)std::max<int64_t>(1, std::min<int64_t>(octs_cap, ((int64_t)tile_y + 7) / 8));
        const int rows_per_panel = octs * 8;
        // panels: contiguous runs of non-empty rows (keeps the column locality of
        // neighbouring rows); inside a panel rows are ranked by length so that the
        // 8 groups of a wave work on rows of similar length in the same slot
        std::vector<int32_t> ne;
        ne.reserve((size_t)I.rows_touched);
        for (int64_t r = 0; r < n_rows; ++r)
            if (row_ptr[r + 1] > row_ptr[r]) ne.push_back((int32_t)r);
        const int64_t n_panels = ((int64_t)ne.size() + rows_per_panel - 1) / rows_per_panel;
        std::vector<int32_t> slot_row((size_t)n_panels * pv.S * pv.NWAVES * 8, -1);
        std::vector<int32_t> panel_tiles((size_t)n_panels * 2, 0);
        parallel_ranges(n_panels, 4, [&](int64_t pb, int64_t pe, int) {
            std::vector<int32_t> rk;
            for (int64_t p = pb; p < pe; ++p) {
                const int64_t b = p * rows_per_panel, e = std::min<int64_t>(b + rows_per_panel, (int64_t)ne.size());
                rk.assign(ne.begin() + b, ne.begin() + e);
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
        if (d_row_ptr_borrowed) {
            P->d_row_ptr = d_row_ptr_borrowed;
        } else {
            int32_t *d = nullptr;
            HIP_TRY(hipMalloc((void **)&d, (size_t)(n_rows + 1) * 4));
            HIP_TRY(hipMemcpy(d, row_ptr, (size_t)(n_rows + 1) * 4, hipMemcpyHostToDevice));
            dev_bytes += (n_rows + 1) * 4;
            P->d_row_ptr = d; P->own_row_ptr = true;
        }
        if (int rc = upload(&P->d_slot_row, slot_row, &dev_bytes)) return rc;
        if (int rc = upload(&P->d_panel_tiles, panel_tiles, &dev_bytes)) return rc;
        P->n_panels = (int32_t)n_panels;
        hipDeviceProp_t prop;
        HIP_TRY(hipGetDeviceProperties(&prop, 0));
        const int cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        I.tile_size_x = x; I.tile_size_y = rows_per_panel; I.k_slice = ks;
        I.n_col_tiles = (int32_t)((n_cols + x - 1) / x); I.n_row_panels = (int32_t)n_panels;
        I.n_blocks = 0;
        for (int64_t p = 0; p < n_panels; ++p) I.n_blocks += panel_tiles[2 * p + 1] - panel_tiles[2 * p] + 1;
        I.lanes_per_nnz = 8;
        I.grid = (int32_t)std::max<int64_t>(1, std::min<int64_t>(cus, n_panels));
        I.block = pv.NWAVES * 64;
        I.lds_bytes = x * ks * 4;
        HIP_TRY(hipFuncSetAttribute((const void *)P->panel_fn, hipFuncAttributeMaxDynamicSharedMemorySize, I.lds_bytes));
        I.device_bytes = dev_bytes;
        I.plan_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        guard.p = nullptr;
        *out = P;
        return SDDMM_OK;
    }
    if (kernel == SDDMM_KERNEL_ROW_GATHER) {
        // segments = non-empty rows
        std::vector<int32_t> seg_end, seg_row;
        seg_end.reserve((size_t)I.rows_touched); seg_row.reserve((size_t)I.rows_touched);
        for (int64_t r = 0; r < n_rows; ++r)
            if (row_ptr[r + 1] > row_ptr[r]) { seg_end.push_back(row_ptr[r + 1]); seg_row.push_back((int32_t)r); }
        P->chunk = 64 * kRowGatherBatchesPerWave * (kRowGatherBlock / 64);
        std::vector<WorkItem> one{{0, (int32_t)nnz, 0, -1}};  // batches are global multiples of 64
        build_batches(one, seg_end.data(), (int64_t)seg_end.size(), batch_seg, batch_mask);
        if (I.rows_touched != n_rows)
            if (int rc = upload(&P->d_seg_row, seg_row, &dev_bytes)) return rc;
        I.tile_size_x = (int32_t)std::min<int64_t>(n_cols, INT32_MAX); I.tile_size_y = (int32_t)std::min<int64_t>(n_rows, INT32_MAX);
        I.n_col_tiles = 1; I.n_row_panels = 1; I.n_blocks = 1;
        I.grid = (int32_t)((nnz + P->chunk - 1) / P->chunk);
        I.block = kRowGatherBlock; I.lds_bytes = 0;
        P->fn = have_fast ? stream_kernel(var, false) : generic_kernel();
    } else {
        int32_t x = tile_x > 0 ? tile_x : fit_x;
        x = std::min(x, fit_x);
        x = (int32_t)std::min<int64_t>(x, std::max<int64_t>(n_cols, 1));
        int32_t y = tile_y > 0 ? tile_y : (int32_t)std::min<int64_t>(std::max<int64_t>(n_rows, 1), INT32_MAX);
        sddmm_tiling T;
        if (int rc = build_tiling(n_rows, n_cols, nnz, row_ptr, col_ind, x, y, T)) return rc;
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
        build_batches(items, T.active_end.data(), (int64_t)T.active_end.size(), batch_seg, batch_mask);
        if (int rc = upload(&P->d_perm, T.tiled_ind, &dev_bytes)) return rc;
        if (int rc = upload(&P->d_seg_row, T.active_row, &dev_bytes)) return rc;
        if (int rc = upload(&P->d_items, items, &dev_bytes)) return rc;
        P->n_items = (int32_t)items.size();
        I.tile_size_x = x; I.tile_size_y = y; I.n_col_tiles = T.n_tiles;
        I.n_row_panels = (int32_t)((T.max_active_rows + y - 1) / y);
        I.n_blocks = n_blocks;
        hipDeviceProp_t prop;
        HIP_TRY(hipGetDeviceProperties(&prop, 0));
        int cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        I.grid = (int32_t)std::max<int64_t>(1, std::min<int64_t>((int64_t)cus, (int64_t)items.size()));
        I.block = kLdsBlock;
        I.lds_bytes = (int32_t)((int64_t)x * row_bytes);
        P->fn = stream_kernel(var, true);
        HIP_TRY(hipFuncSetAttribute((const void *)P->fn, hipFuncAttributeMaxDynamicSharedMemorySize, I.lds_bytes));
    }
    if (!P->fn) return fail(SDDMM_ERR_ARG, "plan: no kernel for K = %d", K);
    if (int rc = upload(&P->d_batch_seg, batch_seg, &dev_bytes)) return rc;
    if (int rc = upload(&P->d_batch_mask, batch_mask, &dev_bytes)) return rc;
    I.device_bytes = dev_bytes;
    I.plan_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    guard.p = nullptr;
    *out = P;
    return SDDMM_OK;
}

}  // namespace

extern "C" {

int sddmm_plan_create(const sddmm_coo *S, int32_t K, int32_t tile_size_x, int32_t tile_size_y, uint32_t flags,
                      sddmm_plan **out)
{
    if (!S || !out) return fail(SDDMM_ERR_ARG, "sddmm_plan_create: NULL argument");
    *out = nullptr;
    if (S->sorted < 0) const_cast<sddmm_coo *>(S)->sorted = check_sorted(*S) ? 1 : 0;
    if (S->sorted != 1) return fail(SDDMM_ERR_UNSORTED, "sddmm_plan_create: matrix is not (row, col)-sorted; call sddmm_coo_sort_rows");
    try {
        std::vector<int32_t> rp;
        build_row_ptr(*S, rp);
        return make_plan(S->n_rows, S->n_cols, S->nnz, rp.data(), S->cols.data(), S->vals.data(), nullptr, nullptr, K,
                         tile_size_x, tile_size_y, flags, out);
    } catch (const std::bad_alloc &) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_create: out of host memory");
    }
}

int sddmm_plan_create_device(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                             const int32_t *d_col_ind, int32_t K, int32_t tile_size_x, int32_t tile_size_y,
                             uint32_t flags, sddmm_plan **out)
{
    if (!out) return fail(SDDMM_ERR_ARG, "sddmm_plan_create_device: out is NULL");
    *out = nullptr;
    if (n_rows < 0 || n_cols < 0 || nnz < 0 || !d_row_ptr || (nnz > 0 && !d_col_ind))
        return fail(SDDMM_ERR_ARG, "sddmm_plan_create_device: bad sizes or NULL arrays");
    if (nnz >= INT32_MAX - 4096 || n_rows >= INT32_MAX || n_cols >= INT32_MAX)
        return fail(SDDMM_ERR_RANGE, "sddmm_plan_create_device: sizes beyond int32 offsets");
    if (int rc = device_ok()) return rc;
    try {
        std::vector<int32_t> rp((size_t)n_rows + 1), ci((size_t)nnz);
        HIP_TRY(hipMemcpy(rp.data(), d_row_ptr, rp.size() * 4, hipMemcpyDeviceToHost));
        if (nnz) HIP_TRY(hipMemcpy(ci.data(), d_col_ind, ci.size() * 4, hipMemcpyDeviceToHost));
        if (rp[0] != 0 || rp[(size_t)n_rows] != nnz)
            return fail(SDDMM_ERR_ARG, "sddmm_plan_create_device: row_ptr does not span [0, nnz]");
        std::vector<char> bad((size_t)hw_threads() + 1, 0);
        parallel_ranges(n_rows, 1 << 12, [&](int64_t b, int64_t e, int t) {
            for (int64_t r = b; r < e; ++r) {
                if (rp[r + 1] < rp[r]) { bad[t] = 1; return; }
                for (int64_t i = rp[r]; i < rp[r + 1]; ++i) {
                    if (ci[i] < 0 || ci[i] >= n_cols) { bad[t] = 2; return; }
                    if (i > rp[r] && ci[i] < ci[i - 1]) { bad[t] = 3; return; }
                }
            }
        });
        for (char c : bad) {
            if (c == 1) return fail(SDDMM_ERR_ARG, "sddmm_plan_create_device: row_ptr is not monotone");
            if (c == 2) return fail(SDDMM_ERR_RANGE, "sddmm_plan_create_device: a column index lies outside the matrix");
            if (c == 3) return fail(SDDMM_ERR_UNSORTED, "sddmm_plan_create_device: columns are not sorted inside a row");
        }
        return make_plan(n_rows, n_cols, nnz, rp.data(), ci.data(), nullptr, d_row_ptr, d_col_ind, K, tile_size_x, tile_size_y,
                         flags, out);
    } catch (const std::bad_alloc &) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_create_device: out of host memory");
    }
}

int sddmm_plan_get_info(const sddmm_plan *plan, sddmm_plan_info *info)
{
    if (!plan || !info) return fail(SDDMM_ERR_ARG, "sddmm_plan_get_info: NULL argument");
    *info = plan->info;
    return SDDMM_OK;
}

void sddmm_plan_destroy(sddmm_plan *plan) { delete plan; }

int sddmm_execute(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H, float *d_out,
                  void *stream)
{
    if (!plan) return fail(SDDMM_ERR_ARG, "sddmm_execute: plan is NULL");
    const sddmm_plan_info &I = plan->info;
    if (I.nnz == 0) return SDDMM_OK;
    if (!d_W || !d_H || !d_out) return fail(SDDMM_ERR_ARG, "sddmm_execute: NULL device pointer");
    if (((uintptr_t)d_W | (uintptr_t)d_H) & 15u)
        if (I.K % 4 == 0 && (plan->variant.G || I.kernel == SDDMM_KERNEL_PANEL))
            return fail(SDDMM_ERR_ARG, "sddmm_execute: W and H must be 16-byte aligned");
    if (I.kernel == SDDMM_KERNEL_PANEL) {
        PanelArgs pa{};
        pa.row_ptr = plan->d_row_ptr; pa.col_ind = plan->d_col;
        pa.val = d_val ? d_val : plan->d_val;
        pa.W = d_W; pa.H = d_H; pa.out = d_out;
        pa.slot_row = plan->d_slot_row; pa.panel_tiles = plan->d_panel_tiles;
        pa.n_panels = plan->n_panels; pa.tile_x = I.tile_size_x; pa.n_cols = (int32_t)I.n_cols; pa.K = I.K;
        for (int k_off = 0; k_off < I.K; k_off += I.k_slice) {
            pa.k_off = k_off;
            pa.accumulate = k_off > 0;
            hipLaunchKernelGGL(plan->panel_fn, dim3((unsigned)I.grid), dim3((unsigned)I.block), (size_t)I.lds_bytes,
                               (hipStream_t)stream, pa);
        }
        HIP_TRY(hipGetLastError());
        return SDDMM_OK;
    }
    KArgs a{};
    a.col_ind = plan->d_col;
    a.val = d_val ? d_val : plan->d_val;
    a.W = d_W; a.H = d_H; a.out = d_out;
    a.perm = plan->d_perm;
    a.seg_row = plan->d_seg_row;
    a.batch_seg = plan->d_batch_seg;
    a.batch_mask = plan->d_batch_mask;
    a.items = plan->d_items;
    a.n_items = plan->n_items;
    a.nnz = (int32_t)I.nnz;
    a.chunk = plan->chunk;
    a.K = I.K;
    a.tile_x = I.tile_size_x;
    a.n_cols = (int32_t)I.n_cols;
    hipLaunchKernelGGL(plan->fn, dim3((unsigned)I.grid), dim3((unsigned)I.block), (size_t)I.lds_bytes,
                       (hipStream_t)stream, a);
    HIP_TRY(hipGetLastError());
    return SDDMM_OK;
}

int sddmm_gpu(const sddmm_plan *plan, const float *h_W, const float *h_H, float *h_out, float *kernel_ms)
{
    if (!plan || !h_W || !h_H || !h_out) return fail(SDDMM_ERR_ARG, "sddmm_gpu: NULL argument");
    const sddmm_plan_info &I = plan->info;
    float *dW = nullptr, *dH = nullptr, *dO = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    struct Free {
        float *&a, *&b, *&c; hipEvent_t &e0, &e1;
        ~Free() { if (a) (void)hipFree(a); if (b) (void)hipFree(b); if (c) (void)hipFree(c);
                  if (e0) (void)hipEventDestroy(e0); if (e1) (void)hipEventDestroy(e1); }
    } fr{dW, dH, dO, e0, e1};
    const size_t wb = (size_t)std::max<int64_t>(I.n_rows * (int64_t)I.K, 1) * 4, hb = (size_t)std::max<int64_t>(I.n_cols * (int64_t)I.K, 1) * 4;
    const size_t ob = (size_t)std::max<int64_t>(I.nnz, 1) * 4;
    HIP_TRY(hipMalloc((void **)&dW, wb));
    HIP_TRY(hipMalloc((void **)&dH, hb));
    HIP_TRY(hipMalloc((void **)&dO, ob));
    HIP_TRY(hipMemcpy(dW, h_W, (size_t)I.n_rows * I.K * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dH, h_H, (size_t)I.n_cols * I.K * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipEventCreate(&e0));
    HIP_TRY(hipEventCreate(&e1));
    HIP_TRY(hipEventRecord(e0, nullptr));
    if (int rc = sddmm_execute(plan, nullptr, dW, dH, dO, nullptr)) return rc;
    HIP_TRY(hipEventRecord(e1, nullptr));
    HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    if (kernel_ms) *kernel_ms = ms;
    HIP_TRY(hipMemcpy(h_out, dO, (size_t)I.nnz * 4, hipMemcpyDeviceToHost));
    return SDDMM_OK;
}

int sddmm_device_info(int *n_devices, char *arch, int arch_len)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) n = 0;
    if (n_devices) *n_devices = n;
    if (arch && arch_len > 0) {
        arch[0] = 0;
        if (n > 0) {
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, 0) == hipSuccess) {
                strncpy(arch, prop.gcnArchName, (size_t)arch_len - 1);
                arch[arch_len - 1] = 0;
            }
        }
    }
    return SDDMM_OK;
}

}  // extern "C"
