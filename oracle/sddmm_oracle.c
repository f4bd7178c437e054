/*
 * CPU oracle for the SDDMM hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic and the host-side data
 * transformations of the reference program (isratnisa/SDDMM_GPU, HiPC18/src).
 * It exists so that tests can check the HIP path against it and so that the
 * bench can time a CPU baseline.  Nothing in the shipped library links,
 * imports or calls it; only tests, the smoke check and the bench's
 * cpu_baseline leg may.
 *
 * Every function cites the reference lines it follows.  How each one is
 * pinned (none of them by a test of the reference, which has none):
 *   oracle_sddmm_csr / _coo  closed forms (W=H=1, K=1, one-hot H, dense
 *                            S vs a library GEMM, power-of-two scaling),
 *                            fp64 brute force on tiny inputs
 *   oracle_sddmm_residual_csr  the same loop with the last operation
 *                            changed: equals val - oracle_sddmm_csr(val = 1)
 *                            bit for bit (tested), closed form W=H=1
 *   oracle_make_csr,
 *   oracle_rewrite_1d        known answer obtained from the reference's own
 *                            util.h, and oracle/_ref (that header compiled
 *                            as it lies) on random inputs when it is built
 *   oracle_initial           glibc drand48 closed form + known first values,
 *                            and oracle/_ref
 *   oracle_transpose_sort    scipy coo->csr of the transposed triples
 *   oracle_parse_mtx         hand-written files with known contents
 *   oracle_row_softmax,
 *   oracle_spmm_csr          the two forms that surround an SDDMM in its machine-
 *                            learning uses (reference README.md:1); the reference
 *                            has no code for them, so they restate the textbook
 *                            definitions and are pinned by closed forms (equal
 *                            logits -> 1/row length, rows sum to 1, shift
 *                            invariance; one-hot H -> column pick), by
 *                            scipy.sparse (csr @ H) and by fp64 brute force
 */
#define _XOPEN_SOURCE 600
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <stdio.h>
#include <ctype.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ */
/* SDDMM over CSR.  Follows HiPC18/src/sddmm.cu:153-177 (sddmm_CPU_CSR):
 * parallel over rows, per nonzero a sequential left-to-right fp32 sum
 * sm += W[row*k+t]*H[col*k+t], then p[ind] = sm * val[ind].
 * row_ptr here is the ordinary (uncompressed) CSR pointer array.       */
void oracle_sddmm_csr(int64_t n_rows, const int32_t *row_ptr,
                      const int32_t *col_ind, const float *val, int32_t k,
                      const float *W, const float *H, float *p, int nthreads)
{
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
    #pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_rows; ++r) {
        for (int64_t ind = row_ptr[r]; ind < row_ptr[r + 1]; ++ind) {
            const float *w = W + (int64_t)r * k;
            const float *h = H + (int64_t)col_ind[ind] * k;
            float sm = 0.0f; /* built with -ffp-contract=off and no fast-math: order and rounding as written */
            for (int32_t t = 0; t < k; ++t) {
                float prod = w[t] * h[t];
                sm = sm + prod;
            }
            p[ind] = sm * val[ind];
        }
    }
}

/* The residual form val - dot over CSR: the loop of sddmm.cu:153-177 with the
 * last operation changed from sm * val[ind] to val[ind] - sm (the error term
 * of the matrix-factorisation updates that README.md:1 names as the use of
 * SDDMM; the reference has no such function).                              */
void oracle_sddmm_residual_csr(int64_t n_rows, const int32_t *row_ptr,
                               const int32_t *col_ind, const float *val, int32_t k,
                               const float *W, const float *H, float *p, int nthreads)
{
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
    #pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_rows; ++r) {
        for (int64_t ind = row_ptr[r]; ind < row_ptr[r + 1]; ++ind) {
            const float *w = W + (int64_t)r * k;
            const float *h = H + (int64_t)col_ind[ind] * k;
            float sm = 0.0f;
            for (int32_t t = 0; t < k; ++t) {
                float prod = w[t] * h[t];
                sm = sm + prod;
            }
            p[ind] = val[ind] - sm;
        }
    }
}

/* SDDMM over COO.  Follows HiPC18/src/sddmm.cu:180-200 (sddmm_CPU_COO):
 * flat parallel loop over nonzeros, static schedule, sequential fp32 sum.
 * The shipping reference stores p[ind] = sm (the "* val" is commented out,
 * sddmm.cu:192); apply_val != 0 gives p[ind] = sm * val[ind], the form of
 * sddmm.cu:171 that this engine implements.                                */
void oracle_sddmm_coo(int64_t nnz, const int32_t *row_ind,
                      const int32_t *col_ind, const float *val, int32_t k,
                      const float *W, const float *H, float *p, int nthreads,
                      int apply_val)
{
#ifdef _OPENMP
    if (nthreads > 0) { omp_set_dynamic(0); omp_set_num_threads(nthreads); }
#endif
    #pragma omp parallel for
    for (int64_t ind = 0; ind < nnz; ++ind) {
        float sm = 0.0f;
        const float *w = W + (int64_t)row_ind[ind] * k;
        const float *h = H + (int64_t)col_ind[ind] * k;
        for (int32_t t = 0; t < k; ++t)
            sm += w[t] * h[t];
        p[ind] = apply_val ? sm * val[ind] : sm;
    }
}

/* Same loop as oracle_sddmm_coo, timed the way the reference times it
 * (omp_get_wtime around the loop only, sddmm.cu:182,196).  Returns seconds. */
double oracle_sddmm_coo_timed(int64_t nnz, const int32_t *row_ind,
                              const int32_t *col_ind, const float *val,
                              int32_t k, const float *W, const float *H,
                              float *p, int nthreads, int apply_val)
{
#ifdef _OPENMP
    double t0 = omp_get_wtime();
    oracle_sddmm_coo(nnz, row_ind, col_ind, val, k, W, H, p, nthreads, apply_val);
    return omp_get_wtime() - t0;
#else
    oracle_sddmm_coo(nnz, row_ind, col_ind, val, k, W, H, p, nthreads, apply_val);
    return -1.0;
#endif
}

int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* fp64 companion used for error analysis only: the same product accumulated
 * in double, plus the conditioning term sum_t |w_t*h_t| * |val|.  Not part
 * of the reference; the exact value every fp32 summation order approximates. */
void oracle_sddmm_f64(int64_t nnz, const int32_t *row_ind,
                      const int32_t *col_ind, const float *val, int32_t k,
                      const float *W, const float *H, double *p, double *absp)
{
    #pragma omp parallel for
    for (int64_t ind = 0; ind < nnz; ++ind) {
        double sm = 0.0, am = 0.0;
        const float *w = W + (int64_t)row_ind[ind] * k;
        const float *h = H + (int64_t)col_ind[ind] * k;
        for (int32_t t = 0; t < k; ++t) {
            double pr = (double)w[t] * (double)h[t];
            sm += pr;
            am += pr < 0 ? -pr : pr;
        }
        p[ind] = sm * (double)val[ind];
        if (absp) absp[ind] = am * (val[ind] < 0 ? -(double)val[ind] : (double)val[ind]);
    }
}

/* ------------------------------------------------------------------ */
/* Compressed CSR over the non-empty rows of a row-sorted COO.
 * Follows HiPC18/src/util.h:131-153 (make_CSR): row_holder[h] is the h-th
 * non-empty row, row_ptr[h]..row_ptr[h+1] its range of nonzeros.  Returns
 * the number of non-empty rows.  The reference also stores row_ptr[h+1]
 * once more after the loop (util.h:152); kept, guarded against overflow.  */
int64_t oracle_make_csr(const int32_t *rows, int64_t nnz, int64_t n_rows,
                        int32_t *row_ptr /* n_rows+1 */, int32_t *row_holder /* n_rows */)
{
    int64_t idx = 0, holder = 0;
    row_ptr[0] = 0;
    while (idx < nnz) {
        int32_t r = rows[idx];
        row_holder[holder] = r;
        while (idx < nnz && rows[idx] == r) idx++;
        holder++;
        row_ptr[holder] = (int32_t)idx;
    }
    if (holder + 1 <= n_rows) row_ptr[holder + 1] = (int32_t)idx;
    return holder;
}

/* Column-tile / row-panel reorder.  Follows HiPC18/src/util.h:267-343
 * (rewrite_matrix_1D) in meaning: for each column tile of width ts in
 * ascending order, for each non-empty row in ascending order, the row's
 * nonzeros with col < tile limit are appended (cursor per row), recording
 *   t_rows[i]   tile-local active-row number
 *   t_cols[i]   global column
 *   t_vals[i]   value
 *   t_ind[i]    index in the original order
 *   active_row[tile*n_rows + j]  global row id of the j-th active row
 *   n_actv_row[tile]
 *   last_idx_tile[tile+1]        end offset of the tile
 *   last_idx_block[tile*max_blk + b]  end offset after every actv_row_size
 *                                active rows (the last, partial block too)
 * Differences from the reference, all in places where it reads or writes
 * out of range: the row loop runs over the non-empty rows only (the
 * reference walks holder < n_rows and reads row_ptr past the last non-empty
 * row, util.h:294-300); the first-block slot the reference writes into the
 * next tile's row (util.h:289-292) is not written; the number of tiles is
 * ceil(n_cols/ts) as the loop bound at util.h:283 gives (the constructor
 * sizes one more, util.h:53).  Returns the largest n_actv_row.             */
int32_t oracle_rewrite_1d(int64_t n_rows, int64_t n_cols, int64_t nnz,
                          const int32_t *cols, const float *vals,
                          const int32_t *row_ptr, const int32_t *row_holder,
                          int64_t n_holder, int32_t ts, int32_t actv_row_size,
                          int32_t *t_rows, int32_t *t_cols, float *t_vals,
                          int32_t *t_ind, int32_t *active_row,
                          int32_t *n_actv_row, int32_t *last_idx_tile,
                          int32_t *last_idx_block)
{
    int64_t max_blk = n_rows / actv_row_size + 1;
    int64_t new_idx = 0;
    int32_t max_active = 0;
    int32_t *row_lim = (int32_t *)malloc(sizeof(int32_t) * (size_t)(n_holder > 0 ? n_holder : 1));
    for (int64_t h = 0; h < n_holder; ++h) row_lim[h] = row_ptr[h];
    last_idx_tile[0] = 0;
    int64_t tile = 0;
    for (int64_t tile_lim = ts; tile_lim <= n_cols + ts - 1; tile_lim += ts, ++tile) {
        int32_t block_count = 0, cur_block = 0;
        n_actv_row[tile] = 0;
        for (int64_t h = 0; h < n_holder; ++h) {
            int64_t idx = row_lim[h];
            int64_t start = idx;
            while (idx < row_ptr[h + 1] && cols[idx] < tile_lim) {
                t_ind[new_idx] = (int32_t)idx;
                t_rows[new_idx] = n_actv_row[tile];
                t_cols[new_idx] = cols[idx];
                t_vals[new_idx] = vals[idx];
                new_idx++;
                idx++;
            }
            if (idx != start) {
                active_row[tile * n_rows + n_actv_row[tile]++] = row_holder[h];
                cur_block++;
            }
            row_lim[h] = (int32_t)idx;
            if (cur_block >= actv_row_size) {
                cur_block = 0;
                last_idx_block[tile * max_blk + block_count] = (int32_t)new_idx;
                block_count++;
            }
            if (h == n_holder - 1 && cur_block > 0 && cur_block < actv_row_size)
                last_idx_block[tile * max_blk + block_count] = (int32_t)new_idx;
        }
        if (n_actv_row[tile] > max_active) max_active = n_actv_row[tile];
        last_idx_tile[tile + 1] = (int32_t)new_idx;
    }
    free(row_lim);
    (void)nnz;
    return max_active;
}

/* Dense-factor initialisation of the reference: X[r*k+t] = 0.1*drand48()
 * after srand48(0).  Follows HiPC18/src/util.h:75-81 (initial).           */
void oracle_initial(float *X, int64_t n, int32_t k)
{
    srand48(0L);
    for (int64_t r = 0; r < n; ++r)
        for (int32_t t = 0; t < k; ++t)
            X[r * k + t] = (float)(0.1 * drand48());
}

/* The same sequence from the published recurrence of drand48 (POSIX:
 * X' = (0x5DEECE66D * X + 0xB) mod 2^48, result X'/2^48, seed state after
 * srand48(s) = (s << 16) | 0x330E) -- used to check oracle_initial without
 * relying on the C library.                                               */
void oracle_initial_closed_form(float *X, int64_t n, int32_t k)
{
    uint64_t x = ((uint64_t)0 << 16) | 0x330EULL;
    const uint64_t a = 0x5DEECE66DULL, c = 0xBULL, m = (1ULL << 48) - 1;
    for (int64_t i = 0; i < n * (int64_t)k; ++i) {
        x = (a * x + c) & m;
        X[i] = (float)(0.1 * ((double)x / 281474976710656.0));
    }
}

/* "Conversion from col sorted to row sorted" of the reference.  Follows
 * HiPC18/src/util.h:82-128 (unsorted_make_CSR): builds (col,row,val) tuples,
 * i.e. TRANSPOSES, sorts them lexicographically (ties on (col,row) broken by
 * value, as std::sort on tuples does), and builds row_ptr over the new rows.
 * Outputs are 0-based (the reference rewrites 1-based for its text dump,
 * util.h:105-106).  out_* have nnz entries, row_ptr has new_n_rows+1.       */
typedef struct { int32_t a, b; float v; } oracle_trip;
static int trip_cmp(const void *x, const void *y)
{
    const oracle_trip *p = (const oracle_trip *)x, *q = (const oracle_trip *)y;
    if (p->a != q->a) return p->a < q->a ? -1 : 1;
    if (p->b != q->b) return p->b < q->b ? -1 : 1;
    if (p->v != q->v) return p->v < q->v ? -1 : 1;
    return 0;
}
void oracle_transpose_sort(const int32_t *rows, const int32_t *cols,
                           const float *vals, int64_t nnz, int64_t new_n_rows,
                           int32_t *out_rows, int32_t *out_cols, float *out_vals,
                           int32_t *row_ptr)
{
    oracle_trip *it = (oracle_trip *)malloc(sizeof(oracle_trip) * (size_t)(nnz > 0 ? nnz : 1));
    for (int64_t i = 0; i < nnz; ++i) { it[i].a = cols[i]; it[i].b = rows[i]; it[i].v = vals[i]; }
    qsort(it, (size_t)nnz, sizeof(oracle_trip), trip_cmp);
    int64_t idx = 0;
    row_ptr[0] = 0;
    for (int64_t r = 0; r < new_n_rows; ++r) {
        while (idx < nnz && it[idx].a == r) {
            out_rows[idx] = it[idx].a; out_cols[idx] = it[idx].b; out_vals[idx] = it[idx].v;
            idx++;
        }
        row_ptr[r + 1] = (int32_t)idx;
    }
    free(it);
}

/* Matrix Market text reader with the reference's grammar.  Follows
 * HiPC18/src/sddmm.cu:257-283: skip lines until one whose first character
 * is a digit, read "rows cols nnz" from it, then nnz triples
 * "row col value" (1-based) converted to 0-based.  (The reference keeps
 * only the first token when the very first line already starts with a
 * digit, sddmm.cu:258-266; here the whole size line is always used.)
 * Call with rows==NULL to get the sizes only.  Returns 0 on success.      */
int oracle_parse_mtx(const char *path, int64_t *n_rows, int64_t *n_cols,
                     int64_t *nnz, int32_t *rows, int32_t *cols, float *vals)
{
    FILE *f = fopen(path, "r");
    if (!f) return -1;
    char line[4096];
    int found = 0;
    while (fgets(line, sizeof line, f)) {
        if (isdigit((unsigned char)line[0])) { found = 1; break; }
    }
    long long r, c, z;
    if (!found || sscanf(line, "%lld %lld %lld", &r, &c, &z) != 3) { fclose(f); return -2; }
    *n_rows = r; *n_cols = c; *nnz = z;
    if (rows) {
        for (long long i = 0; i < z; ++i) {
            long long rid, cid; float v;
            if (fscanf(f, "%lld %lld %f", &rid, &cid, &v) != 3) { fclose(f); return -3; }
            rows[i] = (int32_t)(rid - 1); cols[i] = (int32_t)(cid - 1); vals[i] = v;
        }
    }
    fclose(f);
    return 0;
}

/* ------------------------------------------------------------------ */
/* Row-wise softmax over the stored entries of a CSR matrix:
 * out[p] = exp(x[p] - max_r) / sum_{q in row r} exp(x[q] - max_r).
 * The reference has no such code (README.md:1 names the use); this is the
 * definition, accumulated in double and rounded once, so that it can serve as
 * the exact value an fp32 implementation approximates.                   */
void oracle_row_softmax(int64_t n_rows, const int32_t *row_ptr, const float *x, float *out)
{
    #pragma omp parallel for schedule(dynamic, 256)
    for (int64_t r = 0; r < n_rows; ++r) {
        const int64_t b = row_ptr[r], e = row_ptr[r + 1];
        if (e <= b) continue;
        float mx = x[b];
        for (int64_t p = b + 1; p < e; ++p) mx = x[p] > mx ? x[p] : mx;
        double sum = 0.0;
        for (int64_t p = b; p < e; ++p) sum += exp((double)x[p] - (double)mx);
        for (int64_t p = b; p < e; ++p) out[p] = (float)(exp((double)x[p] - (double)mx) / sum);
    }
}

/* Y[r, 0:k] = sum over the row's entries p (in order) of x[p] * H[col_p, 0:k], fp32, sequential:
 * the sparse-times-dense product that follows an SDDMM in attention-like uses.  absy (may be NULL)
 * receives sum |x[p] * H[col_p, t]| in double, the conditioning term for error bounds.            */
void oracle_spmm_csr(int64_t n_rows, const int32_t *row_ptr, const int32_t *col_ind, const float *x, int32_t k,
                     const float *H, float *Y, double *absy)
{
    #pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_rows; ++r) {
        float *y = Y + r * k;
        for (int32_t t = 0; t < k; ++t) y[t] = 0.0f;
        if (absy) for (int32_t t = 0; t < k; ++t) absy[r * k + t] = 0.0;
        for (int64_t p = row_ptr[r]; p < row_ptr[r + 1]; ++p) {
            const float *h = H + (int64_t)col_ind[p] * k;
            for (int32_t t = 0; t < k; ++t) {
                float prod = x[p] * h[t];
                y[t] = y[t] + prod;
                if (absy) absy[r * k + t] += fabs((double)x[p] * (double)h[t]);
            }
        }
    }
}
