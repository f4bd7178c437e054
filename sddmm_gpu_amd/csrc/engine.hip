// The C entry points of the SDDMM engine for gfx950 (MI355X): plan creation, the execute family,
// values, profiling.  The planner is in planner.hip / planner_tile.hip, plan files in plan_file.hip.
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstring>
#include <new>
#include <unistd.h>
#include "plan.hpp"

using namespace sddmm;

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
