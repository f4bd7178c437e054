// What the planner, the launch code and the plan files of libsddmm_hip.so share: a plan, its launches,
// and the functions that build them.
#pragma once
#include <hip/hip_runtime.h>
#include "internal.hpp"
#include "kernels.hpp"

#define HIP_TRY(expr)                                                                               \
    do {                                                                                            \
        hipError_t e_ = (expr);                                                                     \
        if (e_ != hipSuccess)                                                                       \
            return sddmm::fail(SDDMM_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
    } while (0)

// One kernel launch of a plan.  A plan is a list of launches over disjoint
// sets of rows; together they write every nonzero's output exactly once.
struct Launch {
    int kind = 0;            // SDDMM_KERNEL_ROW_GATHER / LDS_TILE / PANEL
    sddmm::KernelFn fn = nullptr;   // stream kernels
    sddmm::PanelFn pfn = nullptr;   // panel kernel
    sddmm::TileFn tfn = nullptr;        // tile kernel (values in stream order, first K slice); null: not a tile launch
    sddmm::TileFn tfns[5][4] = {};      // [values in stream order / in sorted order / none / residual epilogue with values
                                 //  in stream order / in sorted order][the only K slice / first of several / a later one /
                                 //  all slices inside one launch (null: no such variant)]
    sddmm::KArgs ka{};
    sddmm::PanelArgs pa{};
    sddmm::TileArgs ta{};
    sddmm::DenseFn dfn = nullptr;       // dense-block kernel; null: not a dense launch
    sddmm::DenseArgs da{};
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
    sddmm::SpmmArgs sa{};
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

namespace sddmm {

constexpr size_t kStreamSlack = 256;  // readable entries behind a tile stream's arrays

// (the word mixer of the pattern hash and of the plan files' checksums)
__host__ __device__ inline uint64_t mix64(uint64_t x)
{
    x ^= x >> 33; x *= 0xff51afd7ed558ccdull; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ull; x ^= x >> 33;
    return x;
}

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

struct DenseBlocks;

// planner.hip
int device_ok();
void default_options(sddmm_plan_options &o);
void apply_env_overrides(sddmm_plan_options &o);  // the environment as an override layer over the caller's options
int resolve_functions(Launch &L);  // looks the launch's kernels up from its descriptor and allows them its LDS size
uint64_t pattern_hash_host(int64_t n_rows, int64_t nnz, const int32_t *row_ptr, const int32_t *col_ind);
int pattern_hash_device(int64_t n_rows, int64_t nnz, const int32_t *d_row_ptr, const int32_t *d_col_ind, uint64_t *out);
void build_batches(const std::vector<WorkItem> &items, const int32_t *seg_end, int64_t n_seg, std::vector<int32_t> &batch_seg,
                   std::vector<uint64_t> &batch_mask);
int64_t list_nnz(const Ctx &c, const std::vector<int32_t> &rows);
int add_row_gather(Ctx &c, const std::vector<int32_t> &rows, bool all_rows);
void assign_workspace(sddmm_plan *P);
int make_plan(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr_all, const int32_t *col_ind_all,
              const float *vals, const int32_t *d_row_ptr_borrowed, const int32_t *d_col_borrowed, int32_t K,
              const sddmm_plan_options &opt_in, sddmm_plan **out);
// planner_tile.hip: the rows' nonzeros in tile order (tiles of x columns), every (row, tile) run padded
int add_tile(Ctx &c, const std::vector<int32_t> &rows_in, int32_t x, int32_t panel_rows, int want_g, int ks,
             sddmm_plan_info *I, bool gather = false, bool x_explicit = false);
}  // namespace sddmm
