// Host-side sparse-matrix container and its conversions: creation, (row, col)
// sort, transposing sort, CSR / compressed-CSR pointers, reference-style dense
// factor initialisation.  Plain C++17 + std::thread; no GPU calls here.
#include "internal.hpp"
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <mutex>
#include <numeric>
#include <string>

namespace sddmm {

static thread_local std::string g_err;

void set_error(const char *fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
}

int fail(int code, const char *fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

int hw_threads()
{
    static int n = [] {
        int v = 0;
        if (const char *e = getenv("SDDMM_NUM_THREADS")) v = atoi(e);
        if (v <= 0) v = (int)std::thread::hardware_concurrency();
        if (v <= 0) v = 1;
        return std::min(v, 64);
    }();
    return n;
}

void parallel_ranges(int64_t n, int64_t grain, const std::function<void(int64_t, int64_t, int)> &f,
                     int *n_used)
{
    int nt = hw_threads();
    if (n < grain * 2) nt = 1;
    nt = (int)std::max<int64_t>(1, std::min<int64_t>(nt, n / std::max<int64_t>(grain, 1)));
    if (n_used) *n_used = nt;
    if (nt == 1) {
        f(0, n, 0);
        return;
    }
    // an exception in a worker (an allocation that fails) is carried to the caller
    std::exception_ptr err;
    std::mutex err_mu;
    std::vector<std::thread> th;
    th.reserve(nt);
    for (int t = 0; t < nt; ++t) {
        int64_t b = n * t / nt, e = n * (t + 1) / nt;
        auto body = [&f, &err, &err_mu, b, e, t] {
            try {
                f(b, e, t);
            } catch (...) {
                std::lock_guard<std::mutex> g(err_mu);
                if (!err) err = std::current_exception();
            }
        };
        try {
            th.emplace_back(body);
        } catch (...) {
            body();  // no thread to be had: this range runs here
        }
    }
    for (auto &x : th) x.join();
    if (err) std::rethrow_exception(err);
}

void parallel_dynamic(int64_t n, int64_t chunk, const std::function<void(int64_t, int64_t, int)> &f)
{
    chunk = std::max<int64_t>(chunk, 1);
    const int nt = (int)std::max<int64_t>(1, std::min<int64_t>(hw_threads(), (n + chunk - 1) / chunk));
    if (nt == 1) {
        if (n > 0) f(0, n, 0);
        return;
    }
    std::atomic<int64_t> next{0};
    std::exception_ptr err;
    std::mutex err_mu;
    std::vector<std::thread> th;
    th.reserve(nt);
    for (int t = 0; t < nt; ++t) {
        auto body = [&, t] {
            try {
                for (;;) {
                    const int64_t b = next.fetch_add(chunk);
                    if (b >= n) break;
                    f(b, std::min(n, b + chunk), t);
                }
            } catch (...) {
                next.store(n);  // the others stop at their next chunk
                std::lock_guard<std::mutex> g(err_mu);
                if (!err) err = std::current_exception();
            }
        };
        try {
            th.emplace_back(body);
        } catch (...) {
            body();  // no thread to be had: the chunks left are taken here
        }
    }
    for (auto &x : th) x.join();
    if (err) std::rethrow_exception(err);
}

bool check_sorted(const sddmm_coo &S)
{
    std::vector<char> bad(hw_threads() + 1, 0);
    parallel_ranges(S.nnz, 1 << 16, [&](int64_t b, int64_t e, int t) {
        for (int64_t i = std::max<int64_t>(b, 1); i < e; ++i) {
            if (S.rows[i] < S.rows[i - 1] || (S.rows[i] == S.rows[i - 1] && S.cols[i] < S.cols[i - 1])) {
                bad[t] = 1;
                return;
            }
        }
    });
    return std::none_of(bad.begin(), bad.end(), [](char c) { return c != 0; });
}

void build_row_ptr(const sddmm_coo &S, std::vector<int32_t> &row_ptr)
{
    row_ptr.assign((size_t)S.n_rows + 1, 0);
    // sorted input: row_ptr[r] = first position whose row >= r
    parallel_ranges(S.nnz, 1 << 16, [&](int64_t b, int64_t e, int) {
        for (int64_t i = b; i < e; ++i) {
            int32_t prev = i == 0 ? -1 : S.rows[i - 1];
            for (int32_t r = prev + 1; r <= S.rows[i]; ++r) row_ptr[r] = (int32_t)i;
        }
    });
    int32_t last = S.nnz ? S.rows[S.nnz - 1] : -1;
    for (int64_t r = (int64_t)last + 1; r <= S.n_rows; ++r) row_ptr[r] = (int32_t)S.nnz;
}

// Stable (row, col) sort: counting sort by row, then each row by column.
static void sort_row_col(sddmm_coo &S)
{
    const int64_t nnz = S.nnz, n_rows = S.n_rows;
    std::vector<int64_t> start((size_t)n_rows + 1, 0);
    for (int64_t i = 0; i < nnz; ++i) start[S.rows[i] + 1]++;
    for (int64_t r = 0; r < n_rows; ++r) start[r + 1] += start[r];
    std::vector<int32_t> ncols((size_t)nnz);
    std::vector<float> nvals((size_t)nnz);
    {
        std::vector<int64_t> cur(start.begin(), start.end() - 1);
        for (int64_t i = 0; i < nnz; ++i) {  // stable scatter
            int64_t d = cur[S.rows[i]]++;
            ncols[d] = S.cols[i];
            nvals[d] = S.vals[i];
        }
    }
    parallel_ranges(n_rows, 256, [&](int64_t rb, int64_t re, int) {
        std::vector<uint64_t> key;
        std::vector<float> tmp;
        for (int64_t r = rb; r < re; ++r) {
            int64_t b = start[r], e = start[r + 1];
            for (int64_t i = b; i < e; ++i) S.rows[i] = (int32_t)r;
            bool ok = true;
            for (int64_t i = b + 1; i < e; ++i)
                if (ncols[i] < ncols[i - 1]) { ok = false; break; }
            if (ok) continue;
            key.resize((size_t)(e - b));
            tmp.assign(nvals.begin() + b, nvals.begin() + e);
            for (int64_t i = b; i < e; ++i) key[i - b] = ((uint64_t)(uint32_t)ncols[i] << 32) | (uint64_t)(i - b);
            std::sort(key.begin(), key.end());  // ties keep file order through the position bits
            for (int64_t i = b; i < e; ++i) {
                ncols[i] = (int32_t)(key[i - b] >> 32);
                nvals[i] = tmp[(size_t)(key[i - b] & 0xffffffffu)];
            }
        }
    });
    S.cols.swap(ncols);
    S.vals.swap(nvals);
    S.sorted = 1;
}

}  // namespace sddmm

using namespace sddmm;

extern "C" {

const char *sddmm_last_error(void) { return g_err.c_str(); }
const char *sddmm_version(void) { return "sddmm-mi355x 0.1 (gfx950)"; }

int sddmm_coo_create(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *rows,
                     const int32_t *cols, const float *vals, sddmm_coo **out)
{
    if (!out) return fail(SDDMM_ERR_ARG, "sddmm_coo_create: out is NULL");
    *out = nullptr;
    if (n_rows < 0 || n_cols < 0 || nnz < 0 || (nnz > 0 && (!rows || !cols)))
        return fail(SDDMM_ERR_ARG, "sddmm_coo_create: bad sizes or NULL index arrays");
    if (n_rows >= INT32_MAX || n_cols >= INT32_MAX || nnz >= INT32_MAX)
        return fail(SDDMM_ERR_RANGE, "sddmm_coo_create: sizes beyond int32 offsets (%lld x %lld, nnz %lld)",
                    (long long)n_rows, (long long)n_cols, (long long)nnz);
    for (int64_t i = 0; i < nnz; ++i)
        if (rows[i] < 0 || rows[i] >= n_rows || cols[i] < 0 || cols[i] >= n_cols)
            return fail(SDDMM_ERR_RANGE, "sddmm_coo_create: entry %lld = (%d, %d) outside %lld x %lld",
                        (long long)i, rows[i], cols[i], (long long)n_rows, (long long)n_cols);
    sddmm_coo *S = new (std::nothrow) sddmm_coo;
    if (!S) return fail(SDDMM_ERR_NOMEM, "sddmm_coo_create: out of memory");
    try {
        S->n_rows = n_rows; S->n_cols = n_cols; S->nnz = nnz;
        S->rows.assign(rows, rows + nnz);
        S->cols.assign(cols, cols + nnz);
        if (vals) S->vals.assign(vals, vals + nnz);
        else S->vals.assign((size_t)nnz, 1.0f);
        S->sorted = check_sorted(*S) ? 1 : 0;
    } catch (const std::exception &e) {
        delete S;
        return fail(SDDMM_ERR_NOMEM, "sddmm_coo_create: %s", e.what());
    }
    *out = S;
    return SDDMM_OK;
}

void sddmm_coo_destroy(sddmm_coo *S) { delete S; }

int sddmm_coo_info(const sddmm_coo *S, int64_t *n_rows, int64_t *n_cols, int64_t *nnz, int *sorted)
{
    if (!S) return fail(SDDMM_ERR_ARG, "sddmm_coo_info: S is NULL");
    if (n_rows) *n_rows = S->n_rows;
    if (n_cols) *n_cols = S->n_cols;
    if (nnz) *nnz = S->nnz;
    if (sorted) *sorted = S->sorted == 1;
    return SDDMM_OK;
}

int sddmm_coo_arrays(const sddmm_coo *S, const int32_t **rows, const int32_t **cols, const float **vals)
{
    if (!S) return fail(SDDMM_ERR_ARG, "sddmm_coo_arrays: S is NULL");
    if (rows) *rows = S->rows.data();
    if (cols) *cols = S->cols.data();
    if (vals) *vals = S->vals.data();
    return SDDMM_OK;
}

int sddmm_coo_sort_rows(sddmm_coo *S)
{
    if (!S) return fail(SDDMM_ERR_ARG, "sddmm_coo_sort_rows: S is NULL");
    if (S->sorted == 1) return SDDMM_OK;
    try {
        sort_row_col(*S);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_coo_sort_rows: %s", e.what());
    }
    return SDDMM_OK;
}

int sddmm_coo_transpose_sort(sddmm_coo *S)
{
    if (!S) return fail(SDDMM_ERR_ARG, "sddmm_coo_transpose_sort: S is NULL");
    S->rows.swap(S->cols);
    std::swap(S->n_rows, S->n_cols);
    S->sorted = 0;
    try {
        S->sorted = check_sorted(*S) ? 1 : 0;
        if (S->sorted == 1) return SDDMM_OK;
        sort_row_col(*S);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_coo_transpose_sort: %s", e.what());
    }
    return SDDMM_OK;
}

static int need_sorted(const sddmm_coo *S, const char *who)
{
    if (!S) return fail(SDDMM_ERR_ARG, "%s: S is NULL", who);
    if (S->sorted != 1) return fail(SDDMM_ERR_UNSORTED, "%s: matrix is not (row, col)-sorted; call sddmm_coo_sort_rows", who);
    return SDDMM_OK;
}

int sddmm_coo_row_ptr(const sddmm_coo *S, int32_t *row_ptr)
{
    if (int rc = need_sorted(S, "sddmm_coo_row_ptr")) return rc;
    if (!row_ptr) return fail(SDDMM_ERR_ARG, "sddmm_coo_row_ptr: row_ptr is NULL");
    try {
        std::vector<int32_t> rp;
        build_row_ptr(*S, rp);
        memcpy(row_ptr, rp.data(), rp.size() * sizeof(int32_t));
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_coo_row_ptr: %s", e.what());
    }
    return SDDMM_OK;
}

int sddmm_coo_compress_rows(const sddmm_coo *S, int32_t *row_ptr, int32_t *row_holder, int64_t *n_nonempty)
{
    if (int rc = need_sorted(S, "sddmm_coo_compress_rows")) return rc;
    if (!row_ptr || !row_holder) return fail(SDDMM_ERR_ARG, "sddmm_coo_compress_rows: NULL output");
    std::vector<int32_t> rp;
    try {
        build_row_ptr(*S, rp);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_coo_compress_rows: %s", e.what());
    }
    int64_t h = 0;
    row_ptr[0] = 0;
    for (int64_t r = 0; r < S->n_rows; ++r) {
        if (rp[r + 1] > rp[r]) {
            row_holder[h] = (int32_t)r;
            row_ptr[++h] = rp[r + 1];
        }
    }
    if (n_nonempty) *n_nonempty = h;
    return SDDMM_OK;
}

// The product's own CPU path: rows dealt to threads in chunks, every nonzero a
// sequential fp32 sum over K (t ascending), scaled by the value last -- the
// arithmetic of sddmm_CPU_CSR, HiPC18/src/sddmm.cu:153-177.
int sddmm_cpu(const sddmm_coo *S, int32_t K, const float *W, const float *H, float *out, int32_t n_threads)
{
    if (int rc = need_sorted(S, "sddmm_cpu")) return rc;
    if (K < 1) return fail(SDDMM_ERR_ARG, "sddmm_cpu: K must be >= 1 (got %d)", K);
    if (S->nnz > 0 && (!W || !H || !out)) return fail(SDDMM_ERR_ARG, "sddmm_cpu: NULL argument");
    if (S->nnz == 0) return SDDMM_OK;
    try {
        const int64_t nnz = S->nnz;
        const int32_t *rows = S->rows.data(), *cols = S->cols.data();
        const float *vals = S->vals.data();
        int nt = n_threads > 0 ? std::min<int>(n_threads, 256) : hw_threads();
        const int64_t chunk = std::max<int64_t>(1024, nnz / (64 * (int64_t)nt));
        nt = (int)std::max<int64_t>(1, std::min<int64_t>(nt, (nnz + chunk - 1) / chunk));
        std::atomic<int64_t> next{0};
        auto work = [&] {
            for (;;) {
                const int64_t b = next.fetch_add(chunk);
                if (b >= nnz) break;
                const int64_t e = std::min(nnz, b + chunk);
                for (int64_t p = b; p < e; ++p) {
                    const float *w = W + (int64_t)rows[p] * K, *h = H + (int64_t)cols[p] * K;
                    float sm = 0.f;
                    for (int32_t t = 0; t < K; ++t) sm += w[t] * h[t];
                    out[p] = sm * vals[p];
                }
            }
        };
        std::vector<std::thread> th;
        th.reserve((size_t)nt);
        for (int t = 1; t < nt; ++t) {
            try {
                th.emplace_back(work);
            } catch (...) {
                break;  // fewer threads: the shared counter hands the chunks to those that run
            }
        }
        work();
        for (auto &x : th) x.join();
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_cpu: %s", e.what());
    }
    return SDDMM_OK;
}

int sddmm_init_reference(float *X, int64_t n, int32_t k)
{
    if (!X || n < 0 || k < 1) return fail(SDDMM_ERR_ARG, "sddmm_init_reference: bad arguments");
    srand48(0L);
    for (int64_t i = 0; i < n * (int64_t)k; ++i) X[i] = (float)(0.1 * drand48());
    return SDDMM_OK;
}

}  // extern "C"
