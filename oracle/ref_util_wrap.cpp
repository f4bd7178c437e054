// Build-time wrapper that compiles the reference's own host header
// (HiPC18/src/util.h, found through -I at build time, never copied) and
// exposes three of its functions with C linkage so tests can compare the
// oracle's restatements against them.  TEST INFRASTRUCTURE ONLY; the output
// goes to oracle/_ref/ and is built only where /root/reference exists.
#include <omp.h>
#include <cstdint>
#include <cstring>
#include "util.h"   // the reference's, via -I/root/reference/HiPC18/src

extern "C" {

// util.h:131-153.  row_ptr has n_rows+2 entries, row_holder n_rows+1; both are
// pre-filled by the caller (row_ptr with nnz) because the reference leaves the
// tail unwritten and rewrite_matrix_1D reads it.  Returns #non-empty rows.
long ref_make_CSR(const int *rows, const int *cols, const float *vals, long nnz,
                  long n_rows, int *row_ptr, int *row_holder)
{
    std::vector<int> r(rows, rows + nnz + 1), c(cols, cols + nnz + 1);
    std::vector<float> v(vals, vals + nnz + 1);   // one padded element: the reference reads rows[nnz]
    make_CSR(r, c, v, nnz, n_rows, row_ptr, row_holder);
    long holder = 0;
    while (holder < n_rows && row_ptr[holder + 1] > row_ptr[holder]) holder++;
    return holder;
}

// util.h:33-66 + 267-343.  Caller passes arrays with one padded element.
// Output arrays are sized by the caller as the TiledMatrix constructor does.
int ref_rewrite_matrix_1D(long n_rows, long n_cols, long nnz, const int *rows,
                          const int *cols, const float *vals, int *row_ptr,
                          int *row_holder, int tile_sizeX, int actv,
                          int *t_rows, int *t_cols, float *t_vals, int *t_ind,
                          int *active_row, int *n_actv_row, int *last_idx_tile,
                          int *last_idx_block, int *ntile_c_out, int *max_blk_out)
{
    actv_row_size = actv;
    Matrix S;
    S.n_rows = n_rows; S.n_cols = n_cols; S.nnz = nnz;
    S.rows.assign(rows, rows + nnz + 1);
    S.cols.assign(cols, cols + nnz + 1);
    S.vals.assign(vals, vals + nnz + 1);
    TiledMatrix tS(S, tile_sizeX, actv);
    tS.max_active_row = 0;
    int ret = rewrite_matrix_1D(S, tS, row_ptr, tile_sizeX, row_holder);
    std::memcpy(t_rows, tS.rows.data(), sizeof(int) * nnz);
    std::memcpy(t_cols, tS.cols.data(), sizeof(int) * nnz);
    std::memcpy(t_vals, tS.vals.data(), sizeof(float) * nnz);
    std::memcpy(t_ind, tS.tiled_ind.data(), sizeof(int) * nnz);
    std::memcpy(active_row, tS.active_row.data(), sizeof(int) * tS.active_row.size());
    std::memcpy(n_actv_row, tS.n_actv_row.data(), sizeof(int) * tS.n_actv_row.size());
    std::memcpy(last_idx_tile, tS.lastIdx_tile.data(), sizeof(int) * tS.lastIdx_tile.size());
    std::memcpy(last_idx_block, tS.lastIdx_block_tile.data(), sizeof(int) * tS.lastIdx_block_tile.size());
    *ntile_c_out = tS.ntile_c;
    *max_blk_out = tS.max_active_block;
    return ret;
}

// util.h:75-81
void ref_initial(float *X, long n, int k)
{
    std::vector<float> v((size_t)n * k);
    initial(v, n, k);
    std::memcpy(X, v.data(), sizeof(float) * v.size());
}

}
