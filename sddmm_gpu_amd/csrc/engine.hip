// Plan construction (stream descriptors for the kernels, upload) and launch
// of the SDDMM engine for gfx950 (MI355X).
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstring>
#include <new>
#include <unistd.h>
#include "internal.hpp"
#include "kernels.hpp"
#include "build_id.h"

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

// One kernel launch of a plan.  A plan is a list of launches over disjoint
// sets of rows; together they write every nonzero's output exactly once.
struct Launch {
    int kind = 0;            // SDDMM_KERNEL_ROW_GATHER / LDS_TILE / PANEL
    KernelFn fn = nullptr;   // stream kernels
    PanelFn pfn = nullptr;   // panel kernel
    TileFn tfn = nullptr;        // tile kernel (values in stream order, first K slice); null: not a tile launch
    TileFn tfns[5][4] = {};      // [values in stream order / in sorted order / none / residual epilogue with values
                                 //  in stream order / in sorted order][the only K slice / first of several / a later one /
                                 //  all slices inside one launch (null: no such variant)]
    KArgs ka{};
    PanelArgs pa{};
    TileArgs ta{};
    DenseFn dfn = nullptr;       // dense-block kernel; null: not a dense launch
    DenseArgs da{};
    float *sval = nullptr;        // the plan's values in stream order (launches that walk a permuted stream)
    const int32_t *perm = nullptr;  // stream position -> sorted position of that launch (null: identity)
    int32_t grid = 0, block = 0, lds = 0, k_slice = 0;
    int32_t tile_g = 0, gather_g = 8;
    int64_t nnz = 0, rows = 0, positions = 0;
    // what the function pointers above were looked up with (they are looked up again when a saved plan is loaded)
    int32_t fn_kind = 0;  // 1 stream kernel (row gather), 2 stream kernel with an LDS tile, 3 tile kernel, 4 panel, 5 dense
    int32_t fn_g = 0, fn_kpl = 0, fn_exact = 0, fn_gather = 0, fn_nwaves = 0;
    int32_t fn_nwm = 0;  // tile kernel: waves per workgroup that run the launch's matrix-core share (0: none)
    int32_t fused_slices = 0;  // sliced tile launch small enough that its K slices run inside one kernel launch
    // Scratch memory of the launch (partial results between K slices; packed operands of the matrix-core share):
    // sizes, and where each lies in a caller's workspace (sddmm_execute_ws); the plan's own copies are in ta
    int64_t part_bytes = 0, hp_bytes = 0, wp_bytes = 0;
    int64_t ws_part = 0, ws_hp = 0, ws_wp = 0;
    // the product Y = X H on this launch's tiles (spmm_stream = 1; sp_on == 0: not built)
    SpmmArgs sa{};
    int32_t sp_on = 0, sp_grid = 0, sp_nwaves = 16;  // (16 waves per workgroup: 1.54 against 1.59 ms with 12 on the recommender shape)
    int64_t sp_part_bytes = 0, ws_sp_part = 0;
};

struct sddmm_plan {
    sddmm_plan_info info{};
    std::vector<Launch> launches;
    struct Owned { void *p; size_t bytes; bool scratch = false; };  // scratch: contents need not be kept (plan files)
    std::vector<Owned> owned;   // device allocations freed with the plan (sizes kept for sddmm_plan_save)
    uint64_t pattern_hash = 0;  // of the CSR pattern the plan was built for (see pattern_hash_host)
    const int32_t *d_row_ptr = nullptr, *d_col = nullptr;
    float *d_val = nullptr;
    int32_t requested_kernel = 0;
    int64_t ws_softmax = 0, ws_bytes = 0;  // workspace layout: the launches' scratch, then the softmax pass's records
    sddmm_plan_options options{};  // what the plan was built with, environment overrides applied
    ~sddmm_plan()
    {
        for (const Owned &o : owned) (void)hipFree(o.p);
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

// Everything the launch builders need.
struct Ctx {
    sddmm_plan *P;
    int64_t n_rows, n_cols, nnz;
    const int32_t *row_ptr, *col_ind;  // host CSR
    const float *vals;                 // host values (indexed by position in the original S) or null
    int32_t K;
    int cus;
    int64_t dev_bytes = 0;
    // The CSR above may be what is left of S after the dense blocks were cut out; orig then maps
    // its positions to positions in the original S (null: the CSR is S itself).  Streams record
    // original positions: that is where outputs go and where values come from.
    const int32_t *orig = nullptr;
    sddmm_plan_options opt{};  // the caller's options with the environment overrides applied
    int32_t pos(int64_t p) const { return orig ? orig[p] : (int32_t)p; }
    float value(int64_t p) const { return vals[orig ? orig[p] : p]; }

    template <class T>
    int up(T **dst, const std::vector<T> &src)
    {
        int rc = upload(dst, src, &dev_bytes);
        if (rc == SDDMM_OK && *dst) P->owned.push_back({(void *)*dst, src.size() * sizeof(T)});
        return rc;
    }
    int need_row_ptr()
    {
        if (P->d_row_ptr) return SDDMM_OK;
        int32_t *d = nullptr;
        HIP_TRY(hipMalloc((void **)&d, (size_t)(n_rows + 1) * 4));
        P->owned.push_back({d, (size_t)(n_rows + 1) * 4});
        HIP_TRY(hipMemcpy(d, row_ptr, (size_t)(n_rows + 1) * 4, hipMemcpyHostToDevice));
        dev_bytes += (n_rows + 1) * 4;
        P->d_row_ptr = d;
        return SDDMM_OK;
    }
};

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
__host__ __device__ inline uint64_t mix64(uint64_t x)
{
    x ^= x >> 33; x *= 0xff51afd7ed558ccdull; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ull; x ^= x >> 33;
    return x;
}
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

constexpr size_t kStreamSlack = 256;  // readable entries behind a tile stream's arrays

// Tile launch: the rows' nonzeros in tile order (tiles of x columns), every
// (row, tile) run padded to a multiple of G stream positions.
int add_tile(Ctx &c, const std::vector<int32_t> &rows_in, int32_t x, int32_t panel_rows, int want_g, int ks,
             sddmm_plan_info *I, bool gather = false, bool x_explicit = false)
{
    // gather: the padded stream in plain row order (one tile as wide as S, one panel),
    // H rows read from global memory instead of an LDS tile
    Launch L;
    L.kind = gather ? SDDMM_KERNEL_ROW_GATHER : SDDMM_KERNEL_LDS_TILE;
    // (gather form over column slabs: the stream lists S slab by slab, so that the H rows one pass
    // gathers come from a range small enough to stay in the last-level cache)
    if (gather) {
        x = (int32_t)std::max<int64_t>(c.n_cols, 1);
        if (c.opt.gather_slab_cols > 0) x = (int32_t)std::min<int64_t>(x, c.opt.gather_slab_cols);
        panel_rows = c.opt.gather_panel_rows > 0 ? (int32_t)std::min<int64_t>(c.opt.gather_panel_rows, INT32_MAX) : INT32_MAX;
    }
    L.rows = (int64_t)rows_in.size();
    const TileVariant tv = pick_tile_variant(ks, want_g);  // ks: K elements per launch (K itself or a slice of it)
    // 12 waves per workgroup measured 2-5 % faster than 16 on slices of 64 and 128, slower on 32
    int nwaves = gather ? 4 : (int)(c.opt.tile_waves > 0 ? c.opt.tile_waves : (ks >= 64 ? 12 : 16));
    if (!gather && nwaves != 12) nwaves = 16;
    if (!tv.G || !tile_kernel(tv, 0, gather, 0, nwaves)) return fail(SDDMM_ERR_ARG, "plan: no tile kernel for K = %d", c.K);
    L.fn_kind = 3; L.fn_g = tv.G; L.fn_kpl = tv.KPL; L.fn_gather = gather; L.fn_nwaves = nwaves;
    const int G = tv.G;
    L.nnz = list_nnz(c, rows_in);
    if (L.nnz == 0) return SDDMM_OK;
    // the kernel addresses W (and, in the gather form, H) rows by 32-bit float4 indices
    if ((int64_t)c.n_rows * (c.K / 4) > (int64_t)UINT32_MAX || (gather && (int64_t)c.n_cols * (c.K / 4) > (int64_t)UINT32_MAX))
        return add_row_gather(c, rows_in, false);
    // Work assignment.  grid2d: every workgroup owns one column tile for good (its H
    // tile is staged once) and one of `shares` row blocks that are the same for all
    // tiles, so the workgroups of different tiles read the same W rows at about the same
    // time and share them in L2.  The tile count is raised to a divisor of the CU count.
    const int assign = (int)(c.opt.tile_assign >= 0 ? c.opt.tile_assign : 2);
    bool grid2d = !gather && assign != 0;
    int shares = 1;
    // xcd_local: workgroup b runs on die b % 8 (round-robin dispatch), each die has its
    // own L2.  All column tiles of a row block are then given to workgroups of ONE die,
    // so that the block's W rows are fetched into one L2 only and the pieces of an
    // output line, which come from different tiles, meet in that L2 before they leave it.
    bool xcd_local = false;
    int xcd_steps = 1;
    if (grid2d) {
        const int64_t n_min = (c.n_cols + x - 1) / x;
        if (n_min <= c.cus) {
            int64_t n2 = n_min;
            while (c.cus % n2) ++n2;
            if (!x_explicit || n2 == n_min) {
                x = (int32_t)std::max<int64_t>(1, (c.n_cols + n2 - 1) / n2);
                const int64_t nt = (c.n_cols + x - 1) / x;
                shares = (int)(c.cus / nt);
                const int64_t per_die = c.cus / 8;
                // (every row block stages every H tile again: with few nonzeros per tile -- less than
                // twice a tile's bytes in index data -- the assignment with the fewest row blocks wins)
                const bool staging_dominates = 8.0 * (double)nt * x * ks * 4 > 2.0 * 12.5 * (double)L.nnz;
                if (assign == 2 && c.cus % 8 == 0 && nt == n2 && (n2 % per_die == 0 || per_die % n2 == 0) &&
                    !(staging_dominates && c.opt.tile_few_blocks != 0)) {
                    xcd_local = true;
                    xcd_steps = (int)std::max<int64_t>(1, n2 / per_die);
                    shares = 8 * (int)std::max<int64_t>(1, per_die / n2);
                }
            } else {
                grid2d = false;  // keep the caller's tile width; equal position ranges balance any tile count
            }
        }
        if (grid2d) panel_rows = INT32_MAX;
    }
    // Matrix-core share (only on request, matrix_rows = 1).  Rows filled to a good part of n_cols leave the
    // stream and are computed as whole 32 x 32 blocks (32 such rows x 32 consecutive columns) by extra
    // waves of the same workgroups (see TileArgs::mf_*).  Whole multiples of 256 rows, so that every die
    // gets the same number of groups of 32.  Measured on the recommender shape at K = 128 it loses: a
    // v_mfma_f32 occupies its SIMD's vector unit for as long as it runs (SQ_VALU_MFMA_COEXEC_CYCLES
    // reads 0 with both kinds of waves resident), so the two kinds of work add up instead of overlapping
    // (vector waves alone 0.38 ms, the MFMA stream alone 0.21 ms, together 0.62 ms; the stream with
    // every row 0.63 ms), and what the matrix cores save per flop goes to the cells of a block that hold
    // no nonzero.
    std::vector<int32_t> mf_rows, rest_rows;
    int mf_nwm = 0;
    int64_t mf_nnz = 0;
    if (xcd_local && !gather && tv.G == 8 && tv.KPL == 4 && ks == c.K && (nwaves == 12 || c.opt.tile_waves == 8) && !c.orig &&
        c.opt.matrix_rows > 0 &&
        c.cus % 8 == 0 && c.n_cols >= 32) {
        const int nwm = c.opt.matrix_waves == 8 ? 8 : 4;
        const int nwv = nwm == 8 || c.opt.tile_waves == 8 ? 8 : 12;
        const int64_t lds_need = (int64_t)x * ks * 4 + kMfLdsExtra + (int64_t)nwm * kMfLdsPerWave;
        const int64_t permille = c.opt.matrix_permille > 0 ? c.opt.matrix_permille : 250;
        const int64_t min_deg = std::max<int64_t>(32, permille * c.n_cols / 1000);
        const int64_t n_cb = (c.n_cols + 31) / 32;
        std::vector<int32_t> heavy;
        for (int32_t r : rows_in)
            if (c.row_ptr[r + 1] - c.row_ptr[r] >= min_deg) heavy.push_back(r);
        std::stable_sort(heavy.begin(), heavy.end(), [&](int32_t u, int32_t v) {
            return c.row_ptr[u + 1] - c.row_ptr[u] > c.row_ptr[v + 1] - c.row_ptr[v];
        });
        heavy.resize(heavy.size() / 256 * 256);  // (the lightest of them stay in the stream)
        const int64_t n_groups = (int64_t)heavy.size() / 32;
        const int64_t h_nnz = list_nnz(c, heavy);
        const bool fits = lds_need <= kLdsMaxBytes && tile_kernel_mf(0, nwv, nwm) != nullptr &&
                          n_groups * n_cb * 256 < ((int64_t)1 << 31) && n_cb < (1 << 17) && n_groups < (1 << 17);
        if (fits && !heavy.empty() && heavy.size() < rows_in.size()) {
            std::vector<uint8_t> is_heavy((size_t)c.n_rows, 0);
            for (int32_t r : heavy) is_heavy[(size_t)r] = 1;
            for (int32_t r : rows_in)
                if (!is_heavy[(size_t)r]) rest_rows.push_back(r);
            mf_rows.swap(heavy);
            mf_nwm = nwm;
            mf_nnz = h_nnz;
            nwaves = nwv;
            L.fn_nwaves = nwaves;
        }
    }
    const std::vector<int32_t> &rows = mf_nwm ? rest_rows : rows_in;
    const int64_t stream_nnz = L.nnz - mf_nnz;
    // panel_local (decided below, once the tiling is known): a matrix with more column tiles than
    // workgroups whose rows touch only a few tiles each (banded shapes) is cut into a few row ranges,
    // and each range is walked from top to bottom by a group of workgroups of one die that hold the
    // tiles the rows at the front touch.
    bool panel_local = false;
    int pl_groups = 0;     // groups of workgroups per die
    int pl_slots = 0;      // workgroups per group (a group works on one row range at a time)
    int64_t block_rows_max = 0;  // most rows in one row block / row range of the 2-D assignment
    int64_t pl_sub = 0;    // batches per piece of an item
    // Short batches (see tile_variant_shorts): the last chunk of a (row, tile) run that holds at
    // most G/2 nonzeros is kept apart from the full chunks, and eight such chunks make a batch of
    // their own, which the kernel runs in half the steps.
    const bool shorts = grid2d && tile_variant_shorts(tv.G, tv.KPL, gather) && c.opt.tile_short_batches != 0;
    // gather form: padding positions are flagged and their results go to a scratch line
    const bool flag_padding = gather && c.opt.gather_sink != 0;
    const bool deal_tiles = c.opt.tile_deal != 0;
    std::vector<uint32_t> btype;
    std::vector<WorkItem> items;
    std::vector<std::pair<int, int32_t>> item_keys;  // (row block, tile) of each entry of items ((-1, -1): an empty turn)
    // The product Y = X H on the same items (spmm_stream = 1; see SpmmArgs): built below, next to the items
    const bool want_spmm = c.opt.spmm_stream > 0 && !gather && !c.orig && mf_nwm == 0 && spmm_tile_supported(ks);
    struct SpmmHost {
        std::vector<WorkItem> items;
        std::vector<int32_t> b_off, b_p0, b_len, row_part_ptr, part_slot;
        std::vector<uint16_t> cols;
        bool built = false;
    } sp;
    // Stream order: row panel by row panel (panel_rows consecutive rows of the list),
    // inside a panel column tile by column tile, inside a tile rows ascending.  A
    // (panel, tile) pair with nonzeros is a "unit"; workgroups that work on the units of
    // one panel at the same time share its W rows in L2.
    if (panel_rows < 1) panel_rows = 1;
    std::vector<int32_t> perm, scol, grow, unit_ptr, unit_tile;
    std::vector<float> sval;
    const size_t guess = (size_t)(L.nnz + L.nnz / 4);
    perm.reserve(guess); scol.reserve(guess); grow.reserve(guess / G + 1);
    if (c.vals) sval.reserve(guess);
    std::vector<int64_t> poff;
    std::vector<int32_t> seg_tile;
    int64_t np = 0;
    int32_t n_tiles_all = 0, n_panels = 0;
    for (size_t rb = 0; rb < rows.size(); rb += (size_t)panel_rows, ++n_panels) {
        const int64_t nr = (int64_t)std::min(rows.size() - rb, (size_t)panel_rows);
        sddmm_tiling T;
        if (int rc = build_tiling(c.n_rows, c.n_cols, c.nnz, c.row_ptr, c.col_ind, x, INT32_MAX, T, rows.data() + rb, nr))
            return rc;
        n_tiles_all = T.n_tiles;
        const int64_t n_seg = (int64_t)T.active_end.size();
        // row-block boundaries of the 2-D assignment: equal shares of the rows' nonzeros
        std::vector<int32_t> cut;
        auto make_cuts = [&](int n_shares) {
            cut.assign((size_t)n_shares + 1, INT32_MAX);
            cut[0] = 0;
            if (!grid2d) return;
            int64_t acc = 0; int sidx = 1;
            for (size_t i = 0; i < rows.size() && sidx < n_shares; ++i) {
                acc += c.row_ptr[rows[i] + 1] - c.row_ptr[rows[i]];
                while (sidx < n_shares && acc >= stream_nnz * sidx / n_shares) cut[sidx++] = (i + 1 < rows.size()) ? rows[i + 1] : INT32_MAX;
            }
        };
        make_cuts(shares);
        auto seg_range = [&](int sh, int32_t j, int64_t *s0, int64_t *s1) {
            const int32_t *ab = T.active_row.data() + T.active_ptr[j], *ae = T.active_row.data() + T.active_ptr[j + 1];
            *s0 = T.active_ptr[j] + (std::lower_bound(ab, ae, cut[sh]) - ab);
            *s1 = T.active_ptr[j] + (std::lower_bound(ab, ae, cut[sh + 1]) - ab);
        };
        // Whole-tile items read a W row once per (row, tile) run, and the workgroups of a die are at
        // different rows of their tiles, so little of W is found in L2 again: n_seg row slices cross
        // the L2 boundary.  When a row touches `live` tiles on average and live workgroups fit on a die,
        // a group of that many workgroups can hold exactly the tiles of the rows it is working on: the
        // rows are cut into 8 x (groups per die) ranges, one per group; inside a range the tiles go,
        // in order, to the group's workgroups; a tile's first row in the range is about where the
        // other workgroups of the group are at that time, so every W row is fetched once per range and
        // found in L2 by the other tiles that need it.
        if (grid2d && !xcd_local && shares == 1 && T.n_tiles > c.cus && c.cus % 8 == 0 && !rows.empty() &&
            (c.opt.tile_runs < 0 || c.opt.tile_runs == 2)) {
            const int per_die = c.cus / 8;
            const int live = (int)((n_seg + (int64_t)rows.size() - 1) / (int64_t)rows.size());
            const int groups = live <= per_die ? per_die / live : 0;
            if (groups >= 1) {
                // tile_size_y (rows per range) asks for more, lower ranges: the groups then take several
                // ranges each, one after the other
                int want = 8 * groups;
                if (c.opt.tile_size_y > 0) {
                    const int64_t ranges = ((int64_t)rows.size() + c.opt.tile_size_y - 1) / c.opt.tile_size_y;
                    want = (int)std::min<int64_t>((int64_t)want * std::max<int64_t>(1, (ranges + want - 1) / want), 1 << 20);
                }
                make_cuts(want);
                int64_t n_it = 0, n_ne = 0;
                for (int32_t j = 0; j < T.n_tiles; ++j) {
                    const int32_t *ab = T.active_row.data() + T.active_ptr[j], *ae = T.active_row.data() + T.active_ptr[j + 1];
                    if (ab == ae) continue;
                    ++n_ne;
                    // (the tile's rows are ascending: it touches the ranges from its first row's to its last row's)
                    const int64_t p0 = std::upper_bound(cut.begin(), cut.end() - 1, *ab) - cut.begin() - 1;
                    const int64_t p1 = std::upper_bound(cut.begin(), cut.end() - 1, *(ae - 1)) - cut.begin() - 1;
                    n_it += p1 - p0 + 1;
                }
                // (every item stages its H tile: the rows' W slices against the tiles staged more than once)
                if (live >= 2 && (c.opt.tile_runs == 2 || (double)n_seg > 1.5 * ((double)rows.size() + (double)(n_it - n_ne) * x))) {
                    shares = want;
                    panel_local = true;
                    pl_groups = groups;
                    pl_slots = per_die / groups;
                    // (banded 2^20, K=512, ms per step by batches per wave and piece: 4 -> 4.37, 8 -> 4.25,
                    // 16 -> 4.24, 32 -> 4.27, 128 -> 4.44; whole tiles in runs of neighbours: 4.56)
                    pl_sub = (int64_t)nwaves * 16;
                } else {
                    make_cuts(shares);
                }
            }
        }
        if (grid2d)
            for (int sh = 0; sh < shares; ++sh)
                block_rows_max = std::max<int64_t>(block_rows_max, std::lower_bound(rows.begin(), rows.end(), cut[(size_t)sh + 1]) -
                                                                   std::lower_bound(rows.begin(), rows.end(), cut[(size_t)sh]));
        auto seg_begin = [&](int32_t j, int64_t sg) { return (sg == T.active_ptr[j]) ? T.tile_ptr[j] : T.active_end[sg - 1]; };
        // Layout with short batches: an item (row block x tile) is a sequence of whole batches.  Its
        // runs are cut into chunks of G positions; a run's last chunk with at most G/2 nonzeros is a
        // short chunk.  Full and short chunks are collected apart, in run order, and every eight of
        // a kind are written out as the item's next batch; what is left of both at the end makes
        // the last batch or two, of the full kind.
        struct ItemLay { int64_t begin, end, batch_base, s0, s1; };
        std::vector<ItemLay> lay;
        if (shorts) {
            if (rb != 0) return fail(SDDMM_ERR_ARG, "plan: short-batch layout with more than one panel");
            constexpr int kPerBatch = 8;  // groups per batch (G == 8)
            lay.assign((size_t)T.n_tiles * shares, ItemLay{0, 0, 0, 0, 0});
            int64_t n_batches = 0;
            for (int32_t j = 0; j < T.n_tiles; ++j) {
                if (T.active_ptr[j + 1] > T.active_ptr[j]) {
                    unit_ptr.push_back((int32_t)np);
                    unit_tile.push_back(j);
                }
                for (int sh = 0; sh < shares; ++sh) {
                    ItemLay &it = lay[(size_t)j * shares + sh];
                    seg_range(sh, j, &it.s0, &it.s1);
                    int64_t nf = 0, ns = 0;
                    for (int64_t sg = it.s0; sg < it.s1; ++sg) {
                        const int64_t len = T.active_end[sg] - seg_begin(j, sg), r = len % G;
                        nf += len / G + (r > G / 2);
                        ns += (r >= 1 && r <= G / 2);
                    }
                    const int64_t n_full_chunks = nf + ns % kPerBatch;
                    it.begin = np; it.batch_base = n_batches;
                    it.end = np + (ns / kPerBatch) * 64 + n_full_chunks * G;
                    n_batches += ns / kPerBatch + (n_full_chunks + kPerBatch - 1) / kPerBatch;
                    np = it.begin + (it.end - it.begin + 63) / 64 * 64;  // items start on whole batches of their own
                    if (np >= INT32_MAX - 4096) return fail(SDDMM_ERR_RANGE, "plan: padded stream beyond int32 offsets");
                }
            }
            perm.assign((size_t)np, 0); scol.assign((size_t)np, 0); grow.assign((size_t)(np / G), 0);
            if (c.vals) sval.assign((size_t)np, 0.f);
            std::vector<uint8_t> is_short((size_t)n_batches, 0);
            const int32_t row_bytes = ks * 4;
            const uint32_t k4 = (uint32_t)(c.K / 4);
            parallel_ranges((int64_t)lay.size(), 1, [&](int64_t ib, int64_t ie, int) {
                struct Chunk { int64_t sg, e0; int cnt; };
                for (int64_t ii = ib; ii < ie; ++ii) {
                    const ItemLay &it = lay[(size_t)ii];
                    const int32_t j = (int32_t)(ii / shares);
                    const int32_t tile_base = (int32_t)((int64_t)j * x);
                    Chunk fq[kPerBatch], sq[kPerBatch];
                    int nfq = 0, nsq = 0;
                    int64_t next = 0;  // the item's next batch
                    // chunk ch -> the G positions from d0 on; mirrored: positions G/2.. repeat 0..G/2-1
                    auto put = [&](const Chunk &ch, int64_t d0, bool mirrored) {
                        const int64_t b = seg_begin(j, ch.sg);
                        const int span = mirrored ? G / 2 : G;
                        int64_t d = d0;
                        for (int i = 0; i < ch.cnt; ++i, ++d) {
                            const int32_t p = T.tiled_ind[b + ch.e0 + i];
                            perm[(size_t)d] = c.pos(p);
                            scol[(size_t)d] = (c.col_ind[p] - tile_base) * row_bytes;
                            if (c.vals) sval[(size_t)d] = c.value(p);
                        }
                        for (; d < d0 + span; ++d) {  // padding repeats the chunk's last nonzero
                            perm[(size_t)d] = perm[(size_t)d - 1]; scol[(size_t)d] = scol[(size_t)d - 1];
                            if (c.vals) sval[(size_t)d] = sval[(size_t)d - 1];
                        }
                        for (; d < d0 + G; ++d) {
                            perm[(size_t)d] = perm[(size_t)d - span]; scol[(size_t)d] = scol[(size_t)d - span];
                            if (c.vals) sval[(size_t)d] = sval[(size_t)d - span];
                        }
                        grow[(size_t)(d0 / G)] = (int32_t)((uint32_t)T.active_row[ch.sg] * k4);
                    };
                    auto emit = [&](const Chunk *q, int n, bool is_s) {
                        const int64_t d0 = it.begin + next * 64;
                        for (int k = 0; k < n; ++k) put(q[k], d0 + (int64_t)k * G, is_s);
                        if (is_s) is_short[(size_t)(it.batch_base + next)] = 1;
                        ++next;
                    };
                    for (int64_t sg = it.s0; sg < it.s1; ++sg) {
                        const int64_t len = T.active_end[sg] - seg_begin(j, sg);
                        const int r = (int)(len % G);
                        for (int64_t e0 = 0; e0 + G <= len; e0 += G) {
                            fq[nfq++] = {sg, e0, G};
                            if (nfq == kPerBatch) { emit(fq, nfq, false); nfq = 0; }
                        }
                        if (r > G / 2) {
                            fq[nfq++] = {sg, len - r, r};
                            if (nfq == kPerBatch) { emit(fq, nfq, false); nfq = 0; }
                        } else if (r >= 1) {
                            sq[nsq++] = {sg, len - r, r};
                            if (nsq == kPerBatch) { emit(sq, nsq, true); nsq = 0; }
                        }
                    }
                    // the rest, as full chunks: at most two batches, the last one possibly partial
                    for (int k = 0; k < nsq; ++k) {
                        fq[nfq++] = sq[k];
                        if (nfq == kPerBatch) { emit(fq, nfq, false); nfq = 0; }
                    }
                    if (nfq) emit(fq, nfq, false);
                }
            });
            btype.assign((size_t)((n_batches + 31) / 32) + 8, 0u);
            for (int64_t b = 0; b < n_batches; ++b)
                if (is_short[(size_t)b]) { btype[(size_t)(b >> 5)] |= 1u << (b & 31); ++c.P->info.short_batches; }
        }
        poff.assign((size_t)n_seg + 1, 0);
        seg_tile.assign((size_t)n_seg, 0);
        poff[0] = np;
        for (int32_t j = 0; j < T.n_tiles && !shorts; ++j) {
            if (T.active_ptr[j + 1] > T.active_ptr[j]) {
                unit_ptr.push_back((int32_t)poff[T.active_ptr[j]]);
                unit_tile.push_back(j);
            }
            for (int64_t s = T.active_ptr[j]; s < T.active_ptr[j + 1]; ++s) {
                const int64_t b = (s == T.active_ptr[j]) ? T.tile_ptr[j] : T.active_end[s - 1];
                const int64_t len = T.active_end[s] - b;
                poff[s + 1] = poff[s] + (len + G - 1) / G * G;
                seg_tile[s] = j;
            }
        }
        const int64_t np_new = shorts ? np : poff[n_seg];
        if (np_new >= INT32_MAX - 4096) return fail(SDDMM_ERR_RANGE, "plan: padded stream beyond int32 offsets");
        perm.resize((size_t)np_new); scol.resize((size_t)np_new); grow.resize((size_t)(np_new / G));
        if (c.vals) sval.resize((size_t)np_new);
        parallel_ranges(shorts ? 0 : n_seg, 1 << 10, [&](int64_t sb, int64_t se, int) {
            for (int64_t s = sb; s < se; ++s) {
                const int32_t j = seg_tile[s];
                const int64_t b = (s == T.active_ptr[j]) ? T.tile_ptr[j] : T.active_end[s - 1];
                const int64_t len = T.active_end[s] - b;
                const int32_t tile_base = (int32_t)((int64_t)j * x);
                const int32_t row_bytes = ks * 4;
                const uint32_t k4 = (uint32_t)(c.K / 4);  // W and H rows in float4
                int64_t d = poff[s];
                for (int64_t i = 0; i < len; ++i, ++d) {
                    const int32_t p = T.tiled_ind[b + i];
                    perm[d] = c.pos(p);
                    // byte offset of the H row inside the LDS tile (gather form: index of its first float4 in H)
                    scol[d] = gather ? (int32_t)((uint32_t)c.col_ind[p] * k4) : (c.col_ind[p] - tile_base) * row_bytes;
                    if (c.vals) sval[d] = c.value(p);
                }
                // padding repeats the run's last nonzero: the kernel stores every position
                // without a test, and a repeat stores the same result at the same place
                for (; d < poff[s + 1]; ++d) {
                    perm[d] = flag_padding ? (int32_t)((uint32_t)perm[d - 1] | 0x80000000u) : perm[d - 1];
                    scol[d] = scol[d - 1];
                    if (c.vals) sval[d] = sval[d - 1];
                }
                for (int64_t g = poff[s] / G; g < poff[s + 1] / G; ++g) grow[g] = (int32_t)((uint32_t)T.active_row[s] * k4);
            }
        });
        np = np_new;
        if (flag_padding) {
            // Gather form: in step I of a batch the 8 groups read the H rows of positions
            // 64 b + 8 g + I.  A padding position there re-reads its own row's last column: one
            // more cache line through the load path, which is what binds this kernel.  Point it
            // at the column another group reads in the same step instead (the same line, merged
            // by the load path), and flag its index so that the result is dropped.
            const int64_t nb64 = (np + 63) / 64;
            parallel_ranges(nb64, 1 << 8, [&](int64_t bb, int64_t be, int) {
                for (int64_t b = bb; b < be; ++b) {
                    const int64_t base = b * 64, lim = std::min<int64_t>(np, base + 64);
                    for (int I = 0; I < G; ++I) {
                        int32_t common = scol[(size_t)base];  // (a group's first position is never padding)
                        for (int64_t d = base + I; d < lim; d += G)
                            if (perm[(size_t)d] >= 0) { common = scol[(size_t)d]; break; }
                        for (int64_t d = base + I; d < lim; d += G)
                            if (perm[(size_t)d] < 0) scol[(size_t)d] = common;
                    }
                }
            });
        }
        auto build_spmm = [&](const std::vector<std::pair<int, int32_t>> &keys) {
            // Runs of every item, longest first, eight to a bundle.  A run's nonzeros are consecutive in the sorted
            // S (one row, consecutive columns), so a group needs the position of the first only.
            struct Run { int32_t p0, len, row, tile_base; };
            const size_t ni = keys.size();
            std::vector<std::vector<Run>> runs(ni);
            std::vector<int64_t> n_bund(ni + 1, 0), n_blk(ni + 1, 0);
            parallel_ranges((int64_t)ni, 1, [&](int64_t ib, int64_t ie, int) {
                for (int64_t k = ib; k < ie; ++k) {
                    const int sh = keys[(size_t)k].first;
                    const int32_t j = keys[(size_t)k].second;
                    if (sh < 0) continue;
                    int64_t s0, s1;
                    seg_range(sh, j, &s0, &s1);
                    auto &rv = runs[(size_t)k];
                    rv.reserve((size_t)(s1 - s0));
                    for (int64_t sg = s0; sg < s1; ++sg) {
                        const int64_t b = seg_begin(j, sg);
                        rv.push_back({T.tiled_ind[(size_t)b], (int32_t)(T.active_end[(size_t)sg] - b), T.active_row[(size_t)sg],
                                      (int32_t)((int64_t)j * x)});
                    }
                    std::stable_sort(rv.begin(), rv.end(), [](const Run &u, const Run &v) { return u.len > v.len; });
                    const int64_t nb = ((int64_t)rv.size() + 7) / 8;
                    int64_t blocks = 0;
                    for (int64_t bb = 0; bb < nb; ++bb) blocks += (rv[(size_t)bb * 8].len + 7) / 8;  // rounds of 8 steps (the bundle's first run is its longest)
                    n_bund[(size_t)k + 1] = nb;
                    n_blk[(size_t)k + 1] = blocks;
                }
            });
            for (size_t k = 0; k < ni; ++k) { n_bund[k + 1] += n_bund[k]; n_blk[k + 1] += n_blk[k]; }
            const int64_t NB = n_bund[ni], NBLK = n_blk[ni];
            if (NB * 8 < INT32_MAX && NBLK * 8 < INT32_MAX) {
                sp.items.resize(ni);
                sp.b_off.assign((size_t)NB + 1, 0);
                sp.b_p0.assign((size_t)NB * 8, 0);
                sp.b_len.assign((size_t)NB * 8, 0);
                sp.cols.assign((size_t)NBLK * 64, 0);
                sp.b_off[(size_t)NB] = (int32_t)NBLK;
                // the rows' partial rows: counted per row, then listed
                std::vector<int32_t> row_index((size_t)c.n_rows, -1);
                for (size_t i = 0; i < rows.size(); ++i) row_index[(size_t)rows[i]] = (int32_t)i;
                sp.row_part_ptr.assign(rows.size() + 1, 0);
                for (size_t k = 0; k < ni; ++k)
                    for (const Run &r : runs[k]) ++sp.row_part_ptr[(size_t)row_index[(size_t)r.row] + 1];
                for (size_t i = 0; i < rows.size(); ++i) sp.row_part_ptr[i + 1] += sp.row_part_ptr[i];
                sp.part_slot.assign((size_t)sp.row_part_ptr[rows.size()], 0);
                std::vector<int32_t> fill_at(sp.row_part_ptr.begin(), sp.row_part_ptr.end() - 1);
                for (size_t k = 0; k < ni; ++k) {  // (in item order: a row's partial rows are listed in the order they are written)
                    const auto &rv = runs[k];
                    for (size_t q = 0; q < rv.size(); ++q)
                        sp.part_slot[(size_t)fill_at[(size_t)row_index[(size_t)rv[q].row]]++] = (int32_t)((n_bund[k] + (int64_t)q / 8) * 8 + (int64_t)q % 8);
                }
                parallel_ranges((int64_t)ni, 1, [&](int64_t ib, int64_t ie, int) {
                    for (int64_t k = ib; k < ie; ++k) {
                        const auto &rv = runs[(size_t)k];
                        sp.items[(size_t)k] = {(int32_t)n_bund[(size_t)k], (int32_t)n_bund[(size_t)k + 1], 0,
                                               keys[(size_t)k].second < 0 ? 0 : keys[(size_t)k].second};
                        int64_t blk = n_blk[(size_t)k];
                        for (int64_t bb = 0; bb * 8 < (int64_t)rv.size(); ++bb) {
                            const int64_t B = n_bund[(size_t)k] + bb;
                            const int n8 = (rv[(size_t)bb * 8].len + 7) / 8;
                            sp.b_off[(size_t)B] = (int32_t)blk;
                            for (int gq = 0; gq < 8 && bb * 8 + gq < (int64_t)rv.size(); ++gq) {
                                const Run &r = rv[(size_t)(bb * 8 + gq)];
                                sp.b_p0[(size_t)B * 8 + gq] = r.p0;
                                sp.b_len[(size_t)B * 8 + gq] = r.len;
                                for (int st = 0; st < n8 * 8; ++st) {  // (beyond the run: its last column again, with x = 0)
                                    const int32_t p = r.p0 + std::min(st, r.len - 1);
                                    sp.cols[((size_t)(blk + st / 8) * 8 + gq) * 8 + st % 8] = (uint16_t)(c.col_ind[p] - r.tile_base);
                                }
                            }
                            blk += n8;
                        }
                    }
                });
                sp.built = true;
            }
        };
        if (grid2d) {
            std::vector<int32_t> tiles_ne;
            for (int32_t j = 0; j < T.n_tiles; ++j) if (T.active_ptr[j + 1] > T.active_ptr[j]) tiles_ne.push_back(j);
            auto item_of = [&](int sh, int32_t j) -> WorkItem {
                if (shorts) {
                    const ItemLay &it = lay[(size_t)j * shares + sh];
                    return {(int32_t)it.begin, (int32_t)it.end, (int32_t)it.batch_base, j};
                }
                int64_t s0, s1;
                seg_range(sh, j, &s0, &s1);
                return {(int32_t)poff[s0], (int32_t)poff[s1], 0, j};
            };
            // (a work item's positions are addressed by 32-bit byte offsets from its start)
            if (np_new > (int64_t)1 << 30) return fail(SDDMM_ERR_RANGE, "plan: more than 2^30 stream positions in one tile launch");
            if (xcd_local) {
                // items[b + step * cus] is what workgroup b does in its step-th turn
                const int per_die = c.cus / 8, nt = T.n_tiles;
                // A workgroup with several turns gets tiles of unequal load: the die's
                // tiles sorted by load are dealt out boustrophedon, heavy with light.
                std::vector<int32_t> deal((size_t)8 * nt);
                if (nt >= per_die)
                    for (int die = 0; die < 8; ++die) {
                        std::vector<std::pair<int64_t, int32_t>> ld((size_t)nt);
                        for (int32_t j = 0; j < nt; ++j) {
                            const WorkItem it = item_of(die, j);
                            ld[(size_t)j] = {-(int64_t)(it.end - it.begin), j};
                        }
                        if (deal_tiles) std::sort(ld.begin(), ld.end());
                        for (int step = 0; step < xcd_steps; ++step)
                            for (int slot = 0; slot < per_die; ++slot)
                                deal[(size_t)die * nt + (size_t)step * per_die + slot] =
                                    ld[(size_t)step * per_die + (step % 2 ? per_die - 1 - slot : slot)].second;
                    }
                for (int step = 0; step < xcd_steps; ++step)
                    for (int b = 0; b < c.cus; ++b) {
                        const int die = b % 8, slot = b / 8;
                        const int sh = nt >= per_die ? die : die + 8 * (slot / nt);
                        const int32_t j = nt >= per_die ? deal[(size_t)die * nt + (size_t)step * per_die + slot] : slot % nt;
                        items.push_back(item_of(sh, j));
                        item_keys.push_back({sh, j});
                    }
            } else if (panel_local) {
                // Range sh belongs to die sh % 8, group (sh / 8) % pl_groups.  Its items, in tile order, go to the
                // group's workgroup that is free first (time counted in stream positions).  The waves of
                // a workgroup split an item into equal contiguous parts, so an item is handed over in
                // pieces of pl_sub batches: the rows a workgroup touches at one time then lie close
                // together.  Pieces of one tile follow each other on the same workgroup (staged once).
                std::vector<std::vector<WorkItem>> seq((size_t)c.cus);
                for (int sh = 0; sh < shares; ++sh) {
                    const int die = sh % 8, base = ((sh / 8) % pl_groups) * pl_slots;
                    std::vector<int64_t> free_at((size_t)pl_slots, 0);
                    for (int32_t j : tiles_ne) {
                        const WorkItem it = item_of(sh, j);
                        if (it.end <= it.begin) continue;
                        const int slot = (int)(std::min_element(free_at.begin(), free_at.end()) - free_at.begin());
                        auto &q = seq[(size_t)((base + slot) * 8 + die)];
                        const int64_t nb = ((int64_t)it.end - it.begin + 63) / 64;
                        for (int64_t k0 = 0; k0 < nb; k0 += pl_sub) {
                            const int64_t k1 = std::min(nb, k0 + pl_sub);
                            q.push_back({(int32_t)(it.begin + k0 * 64), (int32_t)std::min<int64_t>(it.end, it.begin + k1 * 64),
                                         (int32_t)(it.batch_base + (shorts ? k0 : 0)), it.tile});
                        }
                        free_at[(size_t)slot] += (int64_t)it.end - it.begin;
                    }
                }
                size_t turns = 0;
                for (auto &q : seq) turns = std::max(turns, q.size());
                items.assign(turns * (size_t)c.cus, WorkItem{0, 0, 0, 0});
                for (int b = 0; b < c.cus; ++b)
                    for (size_t k = 0; k < seq[(size_t)b].size(); ++k) items[k * (size_t)c.cus + (size_t)b] = seq[(size_t)b][k];
            } else if (shares == 1 && c.cus % 8 == 0 && (int64_t)tiles_ne.size() > c.cus &&
                       c.opt.tile_runs != 0) {
                // More tiles than workgroups (a wide matrix; one item per tile, all rows).  Neighbouring
                // tiles of a banded matrix share most of their rows: each turn gives a run of
                // consecutive tiles to the workgroups of one die (workgroup b runs on die b % 8), so
                // that a W row is fetched into one L2 for all the tiles that need it in that turn,
                // instead of into every die's.  Banded 2^20, K=512: 6.63 -> 5.29 ms, reads across
                // the L2 boundary 44 -> 29.5 GB per step.  (Cutting the rows into blocks that fit L2
                // as well, all workgroups of a die on the same block, was slower, 7.7-10.7 ms: the
                // items get small and every one stages its H tile again.)
                const int per_die = c.cus / 8;
                const int64_t n = (int64_t)tiles_ne.size(), turns = (n + c.cus - 1) / c.cus;
                for (int64_t step = 0; step < turns; ++step)
                    for (int b = 0; b < c.cus; ++b) {
                        const int64_t idx = step * c.cus + (int64_t)(b % 8) * per_die + b / 8;
                        items.push_back(idx < n ? item_of(0, tiles_ne[(size_t)idx]) : WorkItem{0, 0, 0, 0});
                        item_keys.push_back(idx < n ? std::pair<int, int32_t>{0, tiles_ne[(size_t)idx]} : std::pair<int, int32_t>{-1, -1});
                    }
            } else {
                for (int sh = 0; sh < shares; ++sh)
                    for (int32_t j : tiles_ne) { items.push_back(item_of(sh, j)); item_keys.push_back({sh, j}); }
            }
            // the product walks the same (row block, tile) items on the same workgroups
            if (want_spmm && !panel_local && item_keys.size() == items.size()) build_spmm(item_keys);
        } else if (want_spmm && rb == 0 && rows.size() <= (size_t)panel_rows) {
            // (equal position ranges for the SDDMM: the product takes one item per column tile)
            std::vector<std::pair<int, int32_t>> keys;
            for (int32_t j = 0; j < T.n_tiles; ++j)
                if (T.active_ptr[j + 1] > T.active_ptr[j]) keys.push_back({0, j});
            build_spmm(keys);
        }
    }
    unit_ptr.push_back((int32_t)np);
    const int64_t n_blocks = (int64_t)unit_tile.size();
    // The kernel requests index data two batches ahead without clamping: past the last
    // position lie kStreamSlack readable entries whose W row and output position are valid
    // (zero), because the W slice and, in later K slices, the old output of the batch
    // after a wave's last one are requested too (and never used).
    perm.resize((size_t)np + kStreamSlack, 0); scol.resize((size_t)np + kStreamSlack, 0);
    grow.resize((size_t)(np / G) + kStreamSlack, 0);
    if (c.vals) sval.resize((size_t)np + kStreamSlack, 0.f);
    TileArgs &a = L.ta;
    int32_t *d_perm = nullptr, *d_scol = nullptr, *d_grow = nullptr;
    float *d_sval = nullptr;
    int32_t *d_uptr = nullptr, *d_utile = nullptr;
    // the compact stream format of narrow K slices (see TileArgs): at K slices of 32 and 64 the
    // kernel is bound by the bytes it streams (K=32: 0.476 -> 0.411 ms); at 128 it is bound by
    // VALU issue and the 6 extra instructions per batch cost more than the bytes save.  perm
    // stays on the device for sddmm_plan_set_values only.
    const bool compact = !gather && ks / 4 <= 16;
    // (the compact form needs a group's nonzeros at consecutive positions of S: not so in a remainder)
    if (compact && c.orig) return fail(SDDMM_ERR_ARG, "plan: compact tile stream over a remainder matrix");
    if (compact) {
        const int64_t ng = np / G;
        std::vector<uint16_t> scol16((size_t)np + kStreamSlack, 0);
        std::vector<int32_t> pbase((size_t)ng + kStreamSlack, 0);
        const int32_t row_bytes = ks * 4;
        parallel_ranges(ng, 1 << 12, [&](int64_t gb, int64_t ge, int) {
            for (int64_t g = gb; g < ge; ++g) {
                int cnt = 1;
                while (cnt < G && perm[(size_t)(g * G + cnt)] != perm[(size_t)(g * G + cnt - 1)]) ++cnt;
                pbase[(size_t)g] = perm[(size_t)(g * G)];
                grow[(size_t)g] |= cnt - 1;
                for (int i = 0; i < G; ++i) scol16[(size_t)(g * G + i)] = (uint16_t)(scol[(size_t)(g * G + i)] / row_bytes);
            }
        });
        uint16_t *d_scol16 = nullptr;
        int32_t *d_pbase = nullptr;
        if (int rc = c.up(&d_scol16, scol16)) return rc;
        if (int rc = c.up(&d_pbase, pbase)) return rc;
        L.ta.scol16 = d_scol16; L.ta.pbase = d_pbase;
        std::vector<int32_t>().swap(scol);  // not used by the compact kernels
    }
    if (shorts) {
        uint32_t *d_btype = nullptr;
        if (int rc = c.up(&d_btype, btype)) return rc;
        L.ta.btype = d_btype;
    }
    if (int rc = c.up(&d_perm, perm)) return rc;
    if (int rc = c.up(&d_scol, scol)) return rc;
    if (int rc = c.up(&d_grow, grow)) return rc;
    if (int rc = c.up(&d_sval, sval)) return rc;
    if (int rc = c.up(&d_uptr, unit_ptr)) return rc;
    if (int rc = c.up(&d_utile, unit_tile)) return rc;
    a.perm = d_perm; a.scol = d_scol; a.grow = d_grow; a.unit_ptr = d_uptr; a.unit_tile = d_utile;
    L.sval = d_sval; L.perm = d_perm;
    a.n_units = (int32_t)unit_tile.size(); a.tile_x = x; a.n_cols = (int32_t)c.n_cols; a.K = c.K;
    if (ks < c.K) {
        // K slices: the partial results stay in stream order between the slices (coalesced stores and loads); only
        // the last slice writes out.  One fp32 per stream position, owned by the plan: executes of a sliced plan
        // that overlap in time would share it.  (Accumulating through out instead, measured on the same build:
        // banded K=512 5.29 against 4.55 ms; recommender K=256, whose runs of 27 positions make the stores to out
        // nearly as coalesced, 1.746 against 1.729 ms.)
        float *d_part = nullptr;
        const size_t bytes = ((size_t)np + kStreamSlack) * 4;
        HIP_TRY(hipMalloc((void **)&d_part, bytes));
        c.P->owned.push_back({d_part, bytes, true});
        c.dev_bytes += (int64_t)bytes;
        a.part = d_part;
        L.part_bytes = (int64_t)bytes;
        // A small launch costs about as much as its work: its K slices then run inside one kernel launch, every wave
        // over its own positions slice after slice (K=256, ms per step: bag-of-words 0.0328 -> 0.0309; recommender
        // shape at 1.1 M nonzeros 0.0381 -> 0.0345, at 5.3 M 0.1267 -> 0.1218).  Not for large streams, whose
        // workgroups share W rows in L2 by being on the same slice at the same time (99.8 M: 1.710 -> 1.742).
        L.fused_slices = c.opt.fuse_slices >= 0 ? (c.opt.fuse_slices != 0) : (np <= ((int64_t)1 << 23));
    }
    if (gather) {
        float *d_sink = nullptr;
        if (int rc = c.up(&d_sink, std::vector<float>(256 * 64, 0.f))) return rc;
        a.sink = d_sink;
    }
    if (mf_nwm) {
        // Groups of 32 rows in order of length; group k of that order belongs to die k % 8 and is stored as
        // group (k % 8) * Gd + k / 8, so that a die's groups are consecutive.
        const int64_t n_cb = (c.n_cols + 31) / 32;
        const int64_t NG = (int64_t)mf_rows.size() / 32, Gd = NG / 8;
        std::vector<int32_t> slot_rows((size_t)NG * 32);
        for (int64_t k = 0; k < NG; ++k)
            std::copy(mf_rows.begin() + k * 32, mf_rows.begin() + (k + 1) * 32, slot_rows.begin() + ((k % 8) * Gd + k / 8) * 32);
        std::vector<uint2> rowinfo((size_t)(NG * n_cb * 32), make_uint2(0u, 0u));
        parallel_ranges(NG, 1, [&](int64_t gb, int64_t ge, int) {
            for (int64_t g = gb; g < ge; ++g) {
                const int64_t die = g / Gd, k = g - die * Gd;
                uint2 *base = rowinfo.data() + (size_t)(die * Gd * n_cb) * 32;
                for (int i = 0; i < 32; ++i) {
                    const int32_t r = slot_rows[(size_t)g * 32 + i];
                    for (int32_t p = c.row_ptr[r]; p < c.row_ptr[r + 1]; ++p) {
                        const int32_t col = c.col_ind[p];
                        uint2 &e = base[((size_t)(col >> 5) * Gd + k) * 32 + i];
                        if (!e.x) e.y = (uint32_t)p;
                        e.x |= 1u << (col & 31);
                    }
                }
            }
        });
        uint2 *d_ri = nullptr;
        int32_t *d_rows = nullptr;
        if (int rc = c.up(&d_ri, rowinfo)) return rc;
        if (int rc = c.up(&d_rows, slot_rows)) return rc;
        float4 *d_hp = nullptr, *d_wp = nullptr;
        const size_t hp_bytes = (size_t)n_cb << 14, wp_bytes = (size_t)NG << 14;
        HIP_TRY(hipMalloc((void **)&d_hp, hp_bytes));
        c.P->owned.push_back({d_hp, hp_bytes, true});
        HIP_TRY(hipMalloc((void **)&d_wp, wp_bytes));
        c.P->owned.push_back({d_wp, wp_bytes, true});
        c.dev_bytes += (int64_t)(hp_bytes + wp_bytes);
        a.mf_hp = d_hp; a.mf_wp = d_wp; a.mf_rowinfo = d_ri; a.mf_rows = d_rows;
        L.hp_bytes = (int64_t)hp_bytes; L.wp_bytes = (int64_t)wp_bytes;
        a.mf_groups = (int32_t)NG; a.mf_n_cb = (int32_t)n_cb;
        a.tile_bytes = (int32_t)((int64_t)x * ks * 4);
        L.fn_nwm = mf_nwm;
        c.P->info.matrix_nnz += mf_nnz;
        c.P->info.matrix_rows += (int64_t)mf_rows.size();
    }
    if (sp.built) {
        SpmmArgs &sa = L.sa;
        WorkItem *d_it = nullptr;
        int32_t *d_off = nullptr, *d_p0 = nullptr, *d_len = nullptr, *d_rpp = nullptr, *d_slot = nullptr, *d_sum = nullptr, *d_gat = nullptr;
        uint16_t *d_cols = nullptr;
        // the rows this launch does not hold (short ones, rows of other launches, rows without entries)
        std::vector<int32_t> others;
        {
            size_t k = 0;
            for (int64_t r = 0; r < c.n_rows; ++r) {
                if (k < rows.size() && rows[k] == (int32_t)r) { ++k; continue; }
                others.push_back((int32_t)r);
            }
            std::stable_sort(others.begin(), others.end(), [&](int32_t u, int32_t v) {
                return c.row_ptr[u + 1] - c.row_ptr[u] > c.row_ptr[v + 1] - c.row_ptr[v];
            });
        }
        if (int rc = c.up(&d_it, sp.items)) return rc;
        if (int rc = c.up(&d_off, sp.b_off)) return rc;
        if (int rc = c.up(&d_p0, sp.b_p0)) return rc;
        if (int rc = c.up(&d_len, sp.b_len)) return rc;
        if (int rc = c.up(&d_cols, sp.cols)) return rc;
        if (int rc = c.up(&d_rpp, sp.row_part_ptr)) return rc;
        if (int rc = c.up(&d_slot, sp.part_slot)) return rc;
        if (int rc = c.up(&d_sum, rows)) return rc;
        if (int rc = c.up(&d_gat, others)) return rc;
        float *d_sp = nullptr;
        const size_t bytes = sp.b_p0.size() * (size_t)ks * 4;
        HIP_TRY(hipMalloc((void **)&d_sp, bytes));
        c.P->owned.push_back({d_sp, bytes, true});
        c.dev_bytes += (int64_t)bytes;
        sa.items = d_it; sa.n_items = (int32_t)sp.items.size(); sa.b_off = d_off; sa.b_p0 = d_p0; sa.b_len = d_len; sa.cols = d_cols;
        sa.part = d_sp; sa.row_part_ptr = d_rpp; sa.part_slot = d_slot; sa.sum_rows = d_sum; sa.n_sum_rows = (int64_t)rows.size();
        sa.gather_rows = d_gat; sa.n_gather_rows = (int64_t)others.size();
        sa.tile_x = x; sa.n_cols = (int32_t)c.n_cols; sa.K = c.K;
        L.sp_on = 1; L.sp_part_bytes = (int64_t)bytes;
        L.sp_grid = (int32_t)std::max<int64_t>(1, std::min<int64_t>((int64_t)c.cus, (int64_t)sp.items.size()));
        c.P->info.spmm_runs += (int64_t)sp.part_slot.size();
    }
    L.grid = (int32_t)std::max<int64_t>(1, std::min<int64_t>((int64_t)c.cus, (np + 4095) / 4096));
    if (grid2d) {
        WorkItem *d_items = nullptr;
        if (int rc = c.up(&d_items, items)) return rc;
        a.items = d_items; a.n_items = (int32_t)items.size();
        L.grid = (int32_t)std::max<int64_t>(1, std::min<int64_t>((int64_t)c.cus, (int64_t)items.size()));
    }
    L.block = (nwaves + mf_nwm) * 64;
    L.lds = gather ? 0 : (int32_t)((int64_t)x * ks * 4);
    if (mf_nwm) {
        L.lds += kMfLdsExtra + mf_nwm * kMfLdsPerWave;
        // (every workgroup's matrix-core waves take a share of their die's pairs: all workgroups must exist)
        if (L.grid != c.cus) return fail(SDDMM_ERR_ARG, "plan: matrix-core share on a launch of %d workgroups", L.grid);
    }
    L.k_slice = ks;
    if (gather) L.grid = (int32_t)std::max<int64_t>(1, (np + 2047) / 2048);
    if (int rc = resolve_functions(L)) return rc;
    if (I) {
        I->tile_size_x = x; I->tile_size_y = grid2d ? (int32_t)std::min<int64_t>(block_rows_max, INT32_MAX) : panel_rows; I->n_col_tiles = n_tiles_all;
        I->n_row_panels = panel_local ? shares : n_panels; I->n_blocks = n_blocks; I->lanes_per_nnz = G; I->lds_bytes = L.lds;
        I->grid = L.grid; I->block = L.block; I->k_slice = ks;
    }
    c.P->info.padded_positions += np;
    L.positions = np; L.tile_g = G;
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

}  // namespace

extern "C" {

void sddmm_plan_options_init(sddmm_plan_options *opt)
{
    if (opt) default_options(*opt);
}

int sddmm_plan_get_options(const sddmm_plan *plan, sddmm_plan_options *opt)
{
    if (!plan || !opt) return fail(SDDMM_ERR_ARG, "sddmm_plan_get_options: NULL argument");
    *opt = plan->options;
    return SDDMM_OK;
}

int sddmm_plan_create_opt(const sddmm_coo *S, int32_t K, const sddmm_plan_options *opt_in, sddmm_plan **out)
{
    if (!S || !out) return fail(SDDMM_ERR_ARG, "sddmm_plan_create: NULL argument");
    *out = nullptr;
    if (S->sorted != 1) return fail(SDDMM_ERR_UNSORTED, "sddmm_plan_create: matrix is not (row, col)-sorted; call sddmm_coo_sort_rows");
    sddmm_plan_options opt;
    default_options(opt);
    if (opt_in) opt = *opt_in;
    try {
        std::vector<int32_t> rp;
        build_row_ptr(*S, rp);
        return make_plan(S->n_rows, S->n_cols, S->nnz, rp.data(), S->cols.data(), S->vals.data(), nullptr, nullptr, K, opt, out);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_create: %s", e.what());
    }
}

int sddmm_plan_create(const sddmm_coo *S, int32_t K, int32_t tile_size_x, int32_t tile_size_y, uint32_t flags,
                      sddmm_plan **out)
{
    sddmm_plan_options opt;
    default_options(opt);
    opt.kernel = (int32_t)(flags & 0xffu); opt.tile_size_x = tile_size_x; opt.tile_size_y = tile_size_y;
    return sddmm_plan_create_opt(S, K, &opt, out);
}

int sddmm_plan_create_device(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                             const int32_t *d_col_ind, int32_t K, int32_t tile_size_x, int32_t tile_size_y,
                             uint32_t flags, sddmm_plan **out)
{
    sddmm_plan_options opt;
    default_options(opt);
    opt.kernel = (int32_t)(flags & 0xffu); opt.tile_size_x = tile_size_x; opt.tile_size_y = tile_size_y;
    return sddmm_plan_create_device_opt(n_rows, n_cols, nnz, d_row_ptr, d_col_ind, K, &opt, out);
}

int sddmm_plan_create_device_opt(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                                 const int32_t *d_col_ind, int32_t K, const sddmm_plan_options *opt_in, sddmm_plan **out)
{
    sddmm_plan_options opt;
    default_options(opt);
    if (opt_in) opt = *opt_in;
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
        return make_plan(n_rows, n_cols, nnz, rp.data(), ci.data(), nullptr, d_row_ptr, d_col_ind, K, opt, out);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_create_device: %s", e.what());
    }
}

int sddmm_plan_get_info(const sddmm_plan *plan, sddmm_plan_info *info)
{
    if (!plan || !info) return fail(SDDMM_ERR_ARG, "sddmm_plan_get_info: NULL argument");
    *info = plan->info;
    return SDDMM_OK;
}

void sddmm_plan_destroy(sddmm_plan *plan) { delete plan; }

static int check_execute_args(const sddmm_plan *plan, const float *d_W, const float *d_H, float *d_out, const char *who)
{
    if (!plan) return fail(SDDMM_ERR_ARG, "%s: plan is NULL", who);
    if (plan->info.nnz == 0) return SDDMM_OK;
    if (!d_W || !d_H || !d_out) return fail(SDDMM_ERR_ARG, "%s: NULL device pointer", who);
    if ((((uintptr_t)d_W | (uintptr_t)d_H) & 15u) && plan->info.K % 4 == 0)
        return fail(SDDMM_ERR_ARG, "%s: W and H must be 16-byte aligned", who);
    return SDDMM_OK;
}

// Issues the kernels of one launch-list entry (one per K slice) on `stream`.
// ws: the caller's workspace (null: the plan's own scratch memory)
static void issue_launch(const sddmm_plan *plan, const Launch &L, const float *d_val, const float *d_W,
                         const float *d_H, float *d_out, hipStream_t stream, int epilogue = SDDMM_EPILOGUE_SCALE, char *ws = nullptr)
{
    const int residual = epilogue == SDDMM_EPILOGUE_RESIDUAL;
    const sddmm_plan_info &I = plan->info;
    const float *val = d_val ? d_val : plan->d_val;
    if (L.kind == SDDMM_KERNEL_PANEL) {
        PanelArgs pa = L.pa;
        pa.row_ptr = plan->d_row_ptr; pa.col_ind = plan->d_col;
        pa.val = val; pa.W = d_W; pa.H = d_H; pa.out = d_out;
        pa.residual = residual;
        for (int k_off = 0; k_off < I.K; k_off += L.k_slice) {
            pa.k_off = k_off;
            pa.accumulate = k_off > 0;
            hipLaunchKernelGGL(L.pfn, dim3((unsigned)L.grid), dim3((unsigned)L.block), (size_t)L.lds, stream, pa);
        }
    } else if (L.dfn) {
        DenseArgs da = L.da;
        da.nz_val = d_val ? nullptr : L.sval;
        da.val = val;
        da.W = d_W; da.H = d_H; da.out = d_out;
        da.residual = residual;
        hipLaunchKernelGGL(L.dfn, dim3((unsigned)L.grid), dim3((unsigned)L.block), 0, stream, da);
    } else if (L.tfn) {
        TileArgs ta = L.ta;
        ta.val = val;
        ta.sval = d_val ? nullptr : L.sval;
        ta.W = d_W; ta.H = d_H; ta.out = d_out;
        ta.nnz = (int32_t)I.nnz;
        if (ws) {
            if (ta.part) ta.part = reinterpret_cast<float *>(ws + L.ws_part);
            if (ta.mf_groups > 0) {
                ta.mf_hp = reinterpret_cast<const float4 *>(ws + L.ws_hp);
                ta.mf_wp = reinterpret_cast<const float4 *>(ws + L.ws_wp);
            }
        }
        if (ta.mf_groups > 0) {  // the matrix-core share reads its operands from packed copies of H and of its W rows
            ta.k_off = 0;
            launch_mf_pack(ta, stream);
        }
        const int vm = residual ? (ta.sval ? 3 : 4) : ta.sval ? 0 : (val ? 1 : 2);
        const bool sliced = L.k_slice < I.K;
        if (sliced && L.fused_slices) {
            ta.k_off = 0; ta.n_slices = I.K / L.k_slice; ta.to_part = 0;
            hipLaunchKernelGGL(L.tfns[vm][3], dim3((unsigned)L.grid), dim3((unsigned)L.block), (size_t)L.lds, stream, ta);
        } else
        for (int k_off = 0; k_off < I.K; k_off += L.k_slice) {
            ta.k_off = k_off;
            ta.to_part = sliced && k_off + L.k_slice < I.K;
            hipLaunchKernelGGL(L.tfns[vm][!sliced ? 0 : k_off == 0 ? 1 : 2], dim3((unsigned)L.grid), dim3((unsigned)L.block), (size_t)L.lds,
                               stream, ta);
        }
    } else {
        KArgs a = L.ka;
        a.col_ind = plan->d_col;
        a.val = val;
        a.sval = d_val ? nullptr : L.sval;
        a.W = d_W; a.H = d_H; a.out = d_out;
        a.residual = residual;
        hipLaunchKernelGGL(L.fn, dim3((unsigned)L.grid), dim3((unsigned)L.block), (size_t)L.lds, stream, a);
    }
}

int sddmm_execute(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H, float *d_out,
                  void *stream)
{
    if (int rc = check_execute_args(plan, d_W, d_H, d_out, "sddmm_execute")) return rc;
    if (plan->info.nnz == 0) return SDDMM_OK;
    for (const Launch &L : plan->launches) issue_launch(plan, L, d_val, d_W, d_H, d_out, (hipStream_t)stream);
    HIP_TRY(hipGetLastError());
    return SDDMM_OK;
}

int sddmm_execute_epilogue(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H, float *d_out,
                           int32_t epilogue, void *stream)
{
    if (int rc = check_execute_args(plan, d_W, d_H, d_out, "sddmm_execute_epilogue")) return rc;
    if (epilogue != SDDMM_EPILOGUE_SCALE && epilogue != SDDMM_EPILOGUE_RESIDUAL)
        return fail(SDDMM_ERR_ARG, "sddmm_execute_epilogue: unknown epilogue %d", (int)epilogue);
    if (epilogue == SDDMM_EPILOGUE_RESIDUAL && !d_val && !plan->d_val && plan->info.nnz > 0)
        return fail(SDDMM_ERR_ARG, "sddmm_execute_epilogue: the residual val - dot needs values (d_val or plan-owned)");
    if (plan->info.nnz == 0) return SDDMM_OK;
    for (const Launch &L : plan->launches) issue_launch(plan, L, d_val, d_W, d_H, d_out, (hipStream_t)stream, epilogue);
    HIP_TRY(hipGetLastError());
    return SDDMM_OK;
}

int sddmm_execute_softmax(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H, float *d_out,
                          void *stream)
{
    if (int rc = sddmm_execute(plan, d_val, d_W, d_H, d_out, stream)) return rc;
    if (plan->info.nnz == 0) return SDDMM_OK;
    if (!plan->d_row_ptr) return fail(SDDMM_ERR_ARG, "sddmm_execute_softmax: the plan holds no row pointers");
    return launch_row_softmax(plan->info.n_rows, plan->d_row_ptr, d_out, d_out, stream, nullptr, 0);
}

int sddmm_plan_workspace_bytes(const sddmm_plan *plan, int64_t *bytes)
{
    if (!plan || !bytes) return fail(SDDMM_ERR_ARG, "sddmm_plan_workspace_bytes: NULL argument");
    *bytes = plan->ws_bytes;
    return SDDMM_OK;
}

int sddmm_execute_ws(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H, float *d_out,
                     int32_t form, void *d_workspace, int64_t workspace_bytes, void *stream)
{
    if (int rc = check_execute_args(plan, d_W, d_H, d_out, "sddmm_execute_ws")) return rc;
    const int32_t epilogue = form & 0xff;
    const bool softmax = (form & SDDMM_FORM_SOFTMAX) != 0;
    if ((form & ~(0xff | SDDMM_FORM_SOFTMAX)) || (epilogue != SDDMM_EPILOGUE_SCALE && epilogue != SDDMM_EPILOGUE_RESIDUAL))
        return fail(SDDMM_ERR_ARG, "sddmm_execute_ws: unknown form %d", (int)form);
    if (epilogue == SDDMM_EPILOGUE_RESIDUAL && !d_val && !plan->d_val && plan->info.nnz > 0)
        return fail(SDDMM_ERR_ARG, "sddmm_execute_ws: the residual val - dot needs values (d_val or plan-owned)");
    if (plan->info.nnz == 0) return SDDMM_OK;
    if (plan->ws_bytes > 0 && (!d_workspace || workspace_bytes < plan->ws_bytes))
        return fail(SDDMM_ERR_ARG, "sddmm_execute_ws: the plan needs a workspace of %lld bytes (sddmm_plan_workspace_bytes)",
                    (long long)plan->ws_bytes);
    if ((uintptr_t)d_workspace & 255u) return fail(SDDMM_ERR_ARG, "sddmm_execute_ws: the workspace must be 256-byte aligned");
    char *ws = static_cast<char *>(d_workspace);
    for (const Launch &L : plan->launches) issue_launch(plan, L, d_val, d_W, d_H, d_out, (hipStream_t)stream, epilogue, ws);
    HIP_TRY(hipGetLastError());
    if (!softmax) return SDDMM_OK;
    if (!plan->d_row_ptr) return fail(SDDMM_ERR_ARG, "sddmm_execute_ws: the plan holds no row pointers");
    return launch_row_softmax(plan->info.n_rows, plan->d_row_ptr, d_out, d_out, stream, ws + plan->ws_softmax, plan->info.nnz);
}

int sddmm_plan_spmm(const sddmm_plan *plan, const float *d_x, const float *d_H, float *d_Y, void *d_workspace,
                    int64_t workspace_bytes, void *stream)
{
    if (!plan) return fail(SDDMM_ERR_ARG, "sddmm_plan_spmm: plan is NULL");
    const sddmm_plan_info &I = plan->info;
    if (I.n_rows == 0) return SDDMM_OK;
    if (!d_Y || (I.nnz > 0 && (!d_x || !d_H))) return fail(SDDMM_ERR_ARG, "sddmm_plan_spmm: NULL device pointer");
    const Launch *Ls = nullptr;
    for (const Launch &L : plan->launches)
        if (L.sp_on) Ls = &L;
    if (!Ls || ((((uintptr_t)d_H) | ((uintptr_t)d_Y)) & 15u)) {
        // no tile stream for the product in this plan: the CSR form, gathering H rows
        if (!plan->d_row_ptr || (I.nnz > 0 && !plan->d_col)) return fail(SDDMM_ERR_ARG, "sddmm_plan_spmm: the plan holds no pattern");
        return sddmm_spmm_csr(I.n_rows, I.n_cols, I.nnz, plan->d_row_ptr, plan->d_col, d_x, I.K, d_H, d_Y, stream);
    }
    if (d_workspace) {
        if (workspace_bytes < plan->ws_bytes) return fail(SDDMM_ERR_ARG, "sddmm_plan_spmm: the plan needs a workspace of %lld bytes", (long long)plan->ws_bytes);
        if ((uintptr_t)d_workspace & 255u) return fail(SDDMM_ERR_ARG, "sddmm_plan_spmm: the workspace must be 256-byte aligned");
    }
    SpmmArgs sa = Ls->sa;
    sa.x = d_x; sa.H = d_H; sa.Y = d_Y;
    sa.row_ptr = plan->d_row_ptr; sa.col_ind = plan->d_col;
    if (d_workspace) sa.part = reinterpret_cast<float *>(static_cast<char *>(d_workspace) + Ls->ws_sp_part);
    for (int k_off = 0; k_off < I.K; k_off += Ls->k_slice) {
        sa.k_off = k_off;
        launch_spmm_slice(sa, Ls->k_slice, Ls->sp_nwaves, Ls->sp_grid, Ls->k_slice * 4 * Ls->ta.tile_x, stream);
    }
    HIP_TRY(hipGetLastError());
    return SDDMM_OK;
}

int sddmm_plan_set_values(sddmm_plan *plan, const float *d_val, void *stream)
{
    if (!plan) return fail(SDDMM_ERR_ARG, "sddmm_plan_set_values: plan is NULL");
    const int64_t nnz = plan->info.nnz;
    if (nnz == 0) return SDDMM_OK;
    if (!d_val) return fail(SDDMM_ERR_ARG, "sddmm_plan_set_values: d_val is NULL");
    if (!plan->d_val) {
        HIP_TRY(hipMalloc((void **)&plan->d_val, (size_t)nnz * 4));
        plan->owned.push_back({plan->d_val, (size_t)nnz * 4});
        plan->info.device_bytes += nnz * 4;
    }
    HIP_TRY(hipMemcpyAsync(plan->d_val, d_val, (size_t)nnz * 4, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    for (Launch &L : plan->launches) {
        if (!L.perm || L.positions <= 0) continue;  // walks S in sorted order: reads d_val directly
        if (!L.sval) {
            HIP_TRY(hipMalloc((void **)&L.sval, ((size_t)L.positions + kStreamSlack) * 4));  // (see add_tile)
            plan->owned.push_back({L.sval, ((size_t)L.positions + kStreamSlack) * 4});
            plan->info.device_bytes += L.positions * 4;
        }
        launch_gather_values(L.perm, plan->d_val, L.sval, L.positions, stream);
    }
    HIP_TRY(hipGetLastError());
    return SDDMM_OK;
}

// ---- plan files -------------------------------------------------------------
// A plan file is the plan's device arrays and launch descriptors under a header with the key it
// was built for.  Device pointers are stored as (allocation number + 1) << 44 | byte offset.
namespace {

struct PlanFileHeader {
    char magic[8];
    uint32_t version, sizeof_launch, sizeof_info, sizeof_options;
    int64_t n_rows, n_cols, nnz;
    int32_t K, requested_kernel;
    uint64_t pattern_hash;
    uint64_t n_allocs, n_launches;
    uint64_t code_row_ptr, code_col, code_val;
    char build[40];          // SDDMM_BUILD_ID of the library that wrote the file: a hash of its sources
    uint64_t meta_checksum;  // over info, options, allocation sizes and launch table as they lie in the file
    uint64_t data_checksum;  // over the arrays, in pieces of kPlanPiece bytes per allocation (see piece_hash)
};
constexpr char kPlanMagic[8] = {'S', 'D', 'D', 'M', 'M', 'P', 'L', 'N'};
constexpr uint32_t kPlanVersion = 4;
constexpr size_t kPlanPiece = (size_t)16 << 20;  // arrays are read, copied and check-summed in pieces of this size

// Hash of one piece of an array: four interleaved multiply-add chains over its 8-byte words (so that a
// thread runs at memory speed), folded with the piece's place in the file.  The file's checksum is the
// wrapping sum of its pieces' hashes, whatever order they are read in.
uint64_t piece_hash(const void *data, size_t n, uint64_t alloc, uint64_t piece)
{
    const unsigned char *b = (const unsigned char *)data;
    uint64_t h[4] = {0x243f6a8885a308d3ull, 0x13198a2e03707344ull, 0xa4093822299f31d0ull, 0x082efa98ec4e6c89ull};
    constexpr uint64_t kMul = 0x9e3779b97f4a7c15ull;
    size_t i = 0;
    for (; i + 32 <= n; i += 32) {
        uint64_t w[4];
        memcpy(w, b + i, 32);
        for (int k = 0; k < 4; ++k) h[k] = (h[k] ^ w[k]) * kMul + (h[k] >> 29);
    }
    uint64_t tail[4] = {0, 0, 0, 0};
    memcpy(tail, b + i, n - i);
    for (int k = 0; k < 4; ++k) h[k] = (h[k] ^ tail[k]) * kMul + (h[k] >> 29);
    uint64_t x = (uint64_t)n;
    for (int k = 0; k < 4; ++k) x = mix64(x ^ h[k]);
    return mix64(x ^ (alloc << 32) ^ piece);
}

// a launch descriptor read from a file must describe a launch this library could have planned
bool launch_plausible(const Launch &L, int64_t nnz)
{
    const int64_t slack = 2 * nnz + (1 << 20);  // padded streams stay well below twice the nonzeros + per-item rounding
    return L.fn_kind >= 1 && L.fn_kind <= 5 && L.grid > 0 && L.grid <= (1 << 24) && L.block >= 64 && L.block <= 1024 &&
           L.block % 64 == 0 && L.lds >= 0 && L.lds <= kLdsMaxBytes && L.nnz >= 0 && L.nnz <= nnz && L.rows >= 0 &&
           L.positions >= 0 && L.positions <= slack + 62 * nnz && L.k_slice >= 0 && L.fn_nwm >= 0 && L.fn_nwm <= 8 &&
           L.ta.n_items >= 0 && L.ta.n_units >= 0 && L.ka.n_items >= 0 && L.ta.mf_groups >= 0 && L.ta.mf_n_cb >= 0;
}
constexpr uint64_t kScratchBit = 1ull << 63;
constexpr uint64_t kBorrowedRowPtr = (1ull << 63) | 1, kBorrowedCol = (1ull << 63) | 2;

// every pointer of a launch that refers to memory the plan owns
void launch_pointer_fields(Launch &L, std::vector<void *> &fields)
{
    fields = {&L.ka.perm, &L.ka.scol, &L.ka.seg_row, &L.ka.batch_seg, &L.ka.batch_mask, &L.ka.items,
            &L.ta.perm, &L.ta.scol, &L.ta.grow, &L.ta.scol16, &L.ta.pbase, &L.ta.btype, &L.ta.part, &L.ta.sink, &L.ta.unit_ptr,
            &L.ta.unit_tile, &L.ta.items, &L.ta.mf_hp, &L.ta.mf_wp, &L.ta.mf_rowinfo, &L.ta.mf_rows,
            &L.sa.items, &L.sa.b_off, &L.sa.b_p0, &L.sa.b_len, &L.sa.cols, &L.sa.part, &L.sa.row_part_ptr, &L.sa.part_slot,
            &L.sa.sum_rows, &L.sa.gather_rows,
            &L.pa.slot_row, &L.pa.panel_tiles,
            &L.da.slot_rows, &L.da.slot_cols, &L.da.slot_range, &L.da.nz_p, &L.da.nz_rc,
            &L.sval, &L.perm};
}

bool encode_pointer(const sddmm_plan *P, const void *p, uint64_t *code)
{
    *code = 0;
    if (!p) return true;
    for (size_t i = 0; i < P->owned.size(); ++i) {
        const char *b = (const char *)P->owned[i].p;
        if ((const char *)p >= b && (const char *)p < b + P->owned[i].bytes) {
            *code = ((uint64_t)(i + 1) << 44) | (uint64_t)((const char *)p - b);
            return true;
        }
    }
    return false;
}

bool decode_pointer(const sddmm_plan *P, uint64_t code, void **p)
{
    *p = nullptr;
    if (!code) return true;
    const uint64_t i = (code >> 44), off = code & ((1ull << 44) - 1);
    if (i < 1 || i > P->owned.size() || off >= P->owned[i - 1].bytes) return false;
    *p = (char *)P->owned[i - 1].p + off;
    return true;
}

bool same_options(const sddmm_plan_options &a, const sddmm_plan_options &b)
{
    // field by field (the structure may hold padding); how the values got there (ignore_env) is not part of the key
    const int la = a.tile_lanes < 0 ? 0 : a.tile_lanes, lb = b.tile_lanes < 0 ? 0 : b.tile_lanes;
    return a.kernel == b.kernel && a.tile_size_x == b.tile_size_x && a.tile_size_y == b.tile_size_y && a.k_slice == b.k_slice &&
           la == lb && a.tile_waves == b.tile_waves && a.tile_assign == b.tile_assign && a.tile_few_blocks == b.tile_few_blocks &&
           a.tile_short_batches == b.tile_short_batches && a.tile_deal == b.tile_deal && a.tile_runs == b.tile_runs && a.fuse_slices == b.fuse_slices &&
           a.gather_lanes == b.gather_lanes && a.gather_padded == b.gather_padded && a.gather_sink == b.gather_sink &&
           a.row_padded == b.row_padded && a.unpadded_tile == b.unpadded_tile && a.dense_blocks == b.dense_blocks &&
           a.dense_permille == b.dense_permille && a.dense_rb_group == b.dense_rb_group &&
           a.matrix_rows == b.matrix_rows && a.matrix_permille == b.matrix_permille && a.matrix_waves == b.matrix_waves &&
           a.spmm_stream == b.spmm_stream &&
           a.gather_slab_cols == b.gather_slab_cols && a.gather_panel_rows == b.gather_panel_rows &&
           a.dense_min_nnz == b.dense_min_nnz && a.panel_bytes == b.panel_bytes && a.short_row_max == b.short_row_max &&
           a.stage_factor == b.stage_factor && a.split_min_nnz == b.split_min_nnz;
}

struct FileCloser { FILE *f; ~FileCloser() { if (f) fclose(f); } };

int load_plan_file(const char *path, int64_t n_rows, int64_t n_cols, int64_t nnz, int32_t K, const sddmm_plan_options *opt_in,
                   const uint64_t *want_hash, const int32_t *d_row_ptr, const int32_t *d_col_ind, sddmm_plan **out)
{
    auto t0 = std::chrono::steady_clock::now();
    if (int rc = device_ok()) return rc;
    FILE *f = fopen(path, "rb");
    if (!f) return fail(SDDMM_ERR_IO, "sddmm_plan_load: cannot open %s", path);
    FileCloser fc{f};
    PlanFileHeader h;
    if (fread(&h, sizeof h, 1, f) != 1 || memcmp(h.magic, kPlanMagic, 8) != 0)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is not a plan file", path);
    h.build[sizeof h.build - 1] = 0;
    if (h.version != kPlanVersion || h.sizeof_launch != sizeof(Launch) || h.sizeof_info != sizeof(sddmm_plan_info) ||
        h.sizeof_options != sizeof(sddmm_plan_options) || strncmp(h.build, SDDMM_BUILD_ID, sizeof h.build - 1) != 0)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s was written by another build of the library (%s, this one is %s)", path,
                    h.build, SDDMM_BUILD_ID);
    if (h.n_rows != n_rows || h.n_cols != n_cols || h.nnz != nnz || h.K != K)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s holds a plan for %lld x %lld, nnz %lld, K %d, not for %lld x %lld, nnz %lld, K %d",
                    path, (long long)h.n_rows, (long long)h.n_cols, (long long)h.nnz, h.K, (long long)n_rows, (long long)n_cols,
                    (long long)nnz, K);
    if (want_hash && *want_hash != h.pattern_hash)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s was built for another sparsity pattern", path);
    if (h.n_allocs > (1u << 20) || h.n_launches > (1u << 16)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged", path);
    sddmm_plan *P = new (std::nothrow) sddmm_plan;
    if (!P) return fail(SDDMM_ERR_NOMEM, "sddmm_plan_load: out of memory");
    struct Guard { sddmm_plan *p; ~Guard() { delete p; } } guard{P};
    if (fread(&P->info, sizeof P->info, 1, f) != 1 || fread(&P->options, sizeof P->options, 1, f) != 1)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is cut short", path);
    if (opt_in) {
        sddmm_plan_options want = *opt_in;
        apply_env_overrides(want);
        if (!same_options(want, P->options))
            return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s was built with other plan options", path);
    }
    std::vector<uint64_t> sizes((size_t)h.n_allocs);
    if (h.n_allocs && fread(sizes.data(), 8, sizes.size(), f) != sizes.size())
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is cut short", path);
    P->launches.resize((size_t)h.n_launches);
    if (h.n_launches && fread((void *)P->launches.data(), sizeof(Launch), P->launches.size(), f) != P->launches.size())
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is cut short", path);
    {
        uint64_t m = piece_hash(&P->info, sizeof P->info, 0, 0) + piece_hash(&P->options, sizeof P->options, 0, 1) +
                     piece_hash(sizes.data(), sizes.size() * 8, 0, 2) +
                     piece_hash((const void *)P->launches.data(), P->launches.size() * sizeof(Launch), 0, 3);
        if (m != h.meta_checksum) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (launch table checksum)", path);
        for (const Launch &L : P->launches)
            if (!launch_plausible(L, nnz)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (launch descriptor)", path);
    }
    // The arrays: pieces of 16 MiB are read (pread) by a few threads, each into its own pair of pinned
    // staging buffers, check-summed there and copied to the device on the thread's own stream as they arrive.
    constexpr size_t kPiece = kPlanPiece;
    const long data_at = ftell(f);
    if (data_at < 0) return fail(SDDMM_ERR_IO, "sddmm_plan_load: cannot seek in %s", path);
    struct Piece { void *dst; uint64_t file_off; size_t n; uint64_t alloc, piece; };
    std::vector<Piece> pieces;
    int64_t total = 0;
    {
        uint64_t at = (uint64_t)data_at, alloc = 0;
        for (uint64_t word : sizes) {
            ++alloc;
            const bool scratch = (word & kScratchBit) != 0;
            const uint64_t bytes = word & ~kScratchBit;
            if (bytes == 0 || bytes > ((uint64_t)1 << 40)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged", path);
            void *d = nullptr;
            HIP_TRY(hipMalloc(&d, bytes));
            P->owned.push_back({d, (size_t)bytes, scratch});
            total += (int64_t)bytes;
            if (scratch) continue;
            for (uint64_t off = 0; off < bytes; off += kPiece)
                pieces.push_back({(char *)d + off, at + off, (size_t)std::min<uint64_t>(kPiece, bytes - off), alloc, off / kPiece});
            at += bytes;
        }
    }
    const int n_readers = (int)std::max<size_t>(1, std::min<size_t>({(size_t)8, (size_t)hw_threads(), pieces.size()}));
    std::vector<int> reader_rc((size_t)n_readers, 0);  // 0 ok, 1 short read, 2 HIP error
    std::vector<uint64_t> reader_sum((size_t)n_readers, 0);
    const int fd = fileno(f);
    {
        std::vector<std::thread> th;
        auto reader = [&](int t) {
                void *stage[2] = {nullptr, nullptr};
                hipEvent_t done[2] = {nullptr, nullptr};
                hipStream_t st = nullptr;
                bool ok = hipStreamCreate(&st) == hipSuccess;
                for (int i = 0; i < 2 && ok; ++i)
                    ok = hipHostMalloc(&stage[i], kPiece, hipHostMallocDefault) == hipSuccess && hipEventCreate(&done[i]) == hipSuccess;
                int turn = 0;
                for (size_t k = (size_t)t; ok && k < pieces.size(); k += (size_t)n_readers, turn ^= 1) {
                    const Piece &pc = pieces[k];
                    if (hipEventSynchronize(done[turn]) != hipSuccess) { ok = false; break; }  // (never recorded: complete)
                    size_t got = 0;
                    while (got < pc.n) {
                        const ssize_t r = pread(fd, (char *)stage[turn] + got, pc.n - got, (off_t)(pc.file_off + got));
                        if (r <= 0) break;
                        got += (size_t)r;
                    }
                    if (got != pc.n) { reader_rc[(size_t)t] = 1; break; }
                    reader_sum[(size_t)t] += piece_hash(stage[turn], pc.n, pc.alloc, pc.piece);
                    ok = hipMemcpyAsync(pc.dst, stage[turn], pc.n, hipMemcpyHostToDevice, st) == hipSuccess &&
                         hipEventRecord(done[turn], st) == hipSuccess;
                }
                if (st) ok = (hipStreamSynchronize(st) == hipSuccess) && ok;
                if (!ok && !reader_rc[(size_t)t]) reader_rc[(size_t)t] = 2;
                for (int i = 0; i < 2; ++i) { if (stage[i]) (void)hipHostFree(stage[i]); if (done[i]) (void)hipEventDestroy(done[i]); }
                if (st) (void)hipStreamDestroy(st);
        };
        // (a thread that cannot be started: its share is read by this one)
        for (int t = 0; t < n_readers; ++t) {
            try {
                th.emplace_back(reader, t);
            } catch (const std::system_error &) {
                reader(t);
            }
        }
        for (auto &x : th) x.join();
    }
    for (int rc : reader_rc) {
        if (rc == 1) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is cut short", path);
        if (rc == 2) return fail(SDDMM_ERR_HIP, "sddmm_plan_load: copying %s to the device failed", path);
    }
    HIP_TRY(hipDeviceSynchronize());
    {
        uint64_t sum = 0;
        for (uint64_t x : reader_sum) sum += x;
        if (sum != h.data_checksum) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (array checksum)", path);
    }
    // pointers
    void *q = nullptr;
    std::vector<void *> fields;
    for (Launch &L : P->launches) {
        launch_pointer_fields(L, fields);
        for (void *field : fields) {
            uint64_t code;
            memcpy(&code, field, 8);
            if (!decode_pointer(P, code, &q)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (bad reference)", path);
            memcpy(field, &q, 8);
        }
        L.ka.col_ind = nullptr; L.ka.val = nullptr; L.ka.W = L.ka.H = nullptr; L.ka.out = nullptr; L.ka.sval = nullptr;
        L.ka.row_ptr = nullptr; L.ka.batch_row = nullptr;
        L.ta.sval = nullptr; L.ta.val = nullptr; L.ta.W = L.ta.H = nullptr; L.ta.out = nullptr;
        L.pa.row_ptr = nullptr; L.pa.col_ind = nullptr; L.pa.val = nullptr; L.pa.W = L.pa.H = nullptr; L.pa.out = nullptr;
        L.da.nz_val = nullptr; L.da.val = nullptr; L.da.W = L.da.H = nullptr; L.da.out = nullptr;
        if (int rc = resolve_functions(L)) return rc;
    }
    auto place = [&](uint64_t code, const int32_t *borrowed, uint64_t marker, const void **dst) -> bool {
        if (code == marker) { *dst = borrowed; return borrowed != nullptr; }
        void *x = nullptr;
        if (!decode_pointer(P, code, &x)) return false;
        *dst = x;
        return true;
    };
    const void *rp = nullptr, *ci = nullptr;
    if (!place(h.code_row_ptr, d_row_ptr, kBorrowedRowPtr, &rp) || !place(h.code_col, d_col_ind, kBorrowedCol, &ci))
        return fail(SDDMM_ERR_ARG, "sddmm_plan_load: %s holds a plan over a device-resident pattern: pass d_row_ptr and d_col_ind "
                                   "(sddmm_plan_load_device)", path);
    P->d_row_ptr = (const int32_t *)rp; P->d_col = (const int32_t *)ci;
    if (!decode_pointer(P, h.code_val, &q)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (bad reference)", path);
    P->d_val = (float *)q;
    P->requested_kernel = h.requested_kernel;
    P->pattern_hash = h.pattern_hash;
    P->info.device_bytes = total;
    assign_workspace(P);
    P->info.plan_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    guard.p = nullptr;
    *out = P;
    return SDDMM_OK;
}

}  // namespace

int sddmm_plan_save(const sddmm_plan *plan, const char *path)
{
    if (!plan || !path) return fail(SDDMM_ERR_ARG, "sddmm_plan_save: NULL argument");
    try {
        PlanFileHeader h;
        memset(&h, 0, sizeof h);
        memcpy(h.magic, kPlanMagic, 8);
        h.version = kPlanVersion; h.sizeof_launch = sizeof(Launch); h.sizeof_info = sizeof(sddmm_plan_info);
        h.sizeof_options = sizeof(sddmm_plan_options);
        h.n_rows = plan->info.n_rows; h.n_cols = plan->info.n_cols; h.nnz = plan->info.nnz; h.K = plan->info.K;
        h.requested_kernel = plan->requested_kernel; h.pattern_hash = plan->pattern_hash;
        h.n_allocs = plan->owned.size(); h.n_launches = plan->launches.size();
        strncpy(h.build, SDDMM_BUILD_ID, sizeof h.build - 1);
        if (!encode_pointer(plan, plan->d_row_ptr, &h.code_row_ptr)) h.code_row_ptr = kBorrowedRowPtr;
        if (!encode_pointer(plan, plan->d_col, &h.code_col)) h.code_col = kBorrowedCol;
        if (!encode_pointer(plan, plan->d_val, &h.code_val)) return fail(SDDMM_ERR_ARG, "sddmm_plan_save: values outside the plan's memory");
        std::vector<Launch> ls(plan->launches);
        std::vector<void *> fields;
        for (Launch &L : ls) {
            launch_pointer_fields(L, fields);
            for (void *field : fields) {
                const void *p;
                memcpy(&p, field, 8);
                uint64_t code;
                if (!encode_pointer(plan, p, &code)) return fail(SDDMM_ERR_ARG, "sddmm_plan_save: a launch refers to memory outside the plan");
                memcpy(field, &code, 8);
            }
            L.fn = nullptr; L.pfn = nullptr; L.tfn = nullptr; L.dfn = nullptr;
            for (auto &row : L.tfns) for (auto &fp : row) fp = nullptr;
        }
        HIP_TRY(hipDeviceSynchronize());  // a set_values still in flight has to land first
        // written under a temporary name and renamed when complete: an interrupted save leaves no file under `path`
        const std::string tmp = std::string(path) + ".tmp";
        FILE *f = fopen(tmp.c_str(), "wb");
        if (!f) return fail(SDDMM_ERR_IO, "sddmm_plan_save: cannot create %s", tmp.c_str());
        struct Unlink { const std::string &p; bool armed = true; ~Unlink() { if (armed) (void)remove(p.c_str()); } } cleanup{tmp};
        bool ok;
        {
            FileCloser fc{f};
            std::vector<uint64_t> sizes;  // (bit 63: scratch, no contents in the file)
            for (const auto &o : plan->owned) sizes.push_back((uint64_t)o.bytes | (o.scratch ? kScratchBit : 0));
            h.meta_checksum = piece_hash(&plan->info, sizeof plan->info, 0, 0) + piece_hash(&plan->options, sizeof plan->options, 0, 1) +
                              piece_hash(sizes.data(), sizes.size() * 8, 0, 2) +
                              piece_hash((const void *)ls.data(), ls.size() * sizeof(Launch), 0, 3);
            ok = fwrite(&h, sizeof h, 1, f) == 1 && fwrite(&plan->info, sizeof plan->info, 1, f) == 1 &&
                 fwrite(&plan->options, sizeof plan->options, 1, f) == 1;
            ok = ok && (sizes.empty() || fwrite(sizes.data(), 8, sizes.size(), f) == sizes.size());
            ok = ok && (ls.empty() || fwrite((const void *)ls.data(), sizeof(Launch), ls.size(), f) == ls.size());
            std::vector<char> buf;
            uint64_t alloc = 0;
            for (const auto &o : plan->owned) {
                ++alloc;
                if (o.scratch) continue;
                for (size_t off = 0; ok && off < o.bytes; off += kPlanPiece) {
                    const size_t n = std::min(kPlanPiece, o.bytes - off);
                    buf.resize(n);
                    HIP_TRY(hipMemcpy(buf.data(), (const char *)o.p + off, n, hipMemcpyDeviceToHost));
                    h.data_checksum += piece_hash(buf.data(), n, alloc, off / kPlanPiece);
                    ok = fwrite(buf.data(), 1, n, f) == n;
                }
            }
            // the header once more, now with the checksum of what followed it
            ok = ok && fseek(f, 0, SEEK_SET) == 0 && fwrite(&h, sizeof h, 1, f) == 1 && fflush(f) == 0;
        }
        if (!ok) return fail(SDDMM_ERR_IO, "sddmm_plan_save: write to %s failed", tmp.c_str());
        if (rename(tmp.c_str(), path) != 0) return fail(SDDMM_ERR_IO, "sddmm_plan_save: cannot rename %s to %s", tmp.c_str(), path);
        cleanup.armed = false;
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_save: %s", e.what());
    }
    return SDDMM_OK;
}

int sddmm_plan_load(const char *path, const sddmm_coo *S, int32_t K, const sddmm_plan_options *opt, sddmm_plan **out)
{
    if (!path || !S || !out) return fail(SDDMM_ERR_ARG, "sddmm_plan_load: NULL argument");
    *out = nullptr;
    if (S->sorted != 1) return fail(SDDMM_ERR_UNSORTED, "sddmm_plan_load: matrix is not (row, col)-sorted");
    try {
        std::vector<int32_t> rp;
        build_row_ptr(*S, rp);
        const uint64_t hash = pattern_hash_host(S->n_rows, S->nnz, rp.data(), S->cols.data());
        return load_plan_file(path, S->n_rows, S->n_cols, S->nnz, K, opt, &hash, nullptr, nullptr, out);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_load: %s", e.what());
    }
}

int sddmm_plan_load_device(const char *path, int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                           const int32_t *d_col_ind, int32_t K, const sddmm_plan_options *opt, sddmm_plan **out)
{
    if (!path || !out) return fail(SDDMM_ERR_ARG, "sddmm_plan_load_device: NULL argument");
    *out = nullptr;
    if (n_rows < 0 || n_cols < 0 || nnz < 0 || !d_row_ptr || (nnz > 0 && !d_col_ind))
        return fail(SDDMM_ERR_ARG, "sddmm_plan_load_device: bad sizes or NULL arrays");
    if (int rc = device_ok()) return rc;
    try {
        uint64_t hash = 0;
        if (int rc = pattern_hash_device(n_rows, nnz, d_row_ptr, d_col_ind, &hash)) return rc;
        return load_plan_file(path, n_rows, n_cols, nnz, K, opt, &hash, d_row_ptr, d_col_ind, out);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_load_device: %s", e.what());
    }
}

int sddmm_plan_launch_count(const sddmm_plan *plan, int32_t *n)
{
    if (!plan || !n) return fail(SDDMM_ERR_ARG, "sddmm_plan_launch_count: NULL argument");
    *n = (int32_t)plan->launches.size();
    return SDDMM_OK;
}

int sddmm_execute_profiled(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H,
                           float *d_out, void *stream, sddmm_launch_profile *prof, int32_t max_prof)
{
    if (int rc = check_execute_args(plan, d_W, d_H, d_out, "sddmm_execute_profiled")) return rc;
    if (!prof || max_prof < (int32_t)plan->launches.size())
        return fail(SDDMM_ERR_ARG, "sddmm_execute_profiled: room for %zu profiles needed", plan->launches.size());
    if (plan->info.nnz == 0) return SDDMM_OK;
    const size_t n = plan->launches.size();
    std::vector<hipEvent_t> ev(n + 1, nullptr);
    struct Ev { std::vector<hipEvent_t> &e; ~Ev() { for (auto x : e) if (x) (void)hipEventDestroy(x); } } guard{ev};
    for (auto &x : ev) HIP_TRY(hipEventCreate(&x));
    HIP_TRY(hipEventRecord(ev[0], (hipStream_t)stream));
    for (size_t i = 0; i < n; ++i) {
        issue_launch(plan, plan->launches[i], d_val, d_W, d_H, d_out, (hipStream_t)stream);
        HIP_TRY(hipEventRecord(ev[i + 1], (hipStream_t)stream));
    }
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipEventSynchronize(ev[n]));
    for (size_t i = 0; i < n; ++i) {
        const Launch &L = plan->launches[i];
        float ms = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms, ev[i], ev[i + 1]));
        prof[i].kernel = L.kind;
        prof[i].lanes_per_nnz = L.dfn ? 0 : L.kind == SDDMM_KERNEL_PANEL ? 8 : (L.tfn ? L.tile_g : L.gather_g);
        prof[i].k_slice = L.k_slice;
        prof[i].n_kernel_launches = (L.k_slice > 0 && L.k_slice < plan->info.K && !L.fused_slices) ? plan->info.K / L.k_slice : 1;
        prof[i].nnz = L.nnz;
        prof[i].rows = L.rows;
        prof[i].stream_positions = L.positions;
        prof[i].ms = ms;
    }
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
