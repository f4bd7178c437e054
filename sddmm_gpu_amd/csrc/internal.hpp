// Internal definitions shared by the host-side sources of libsddmm_hip.so.
#pragma once
#include <cstdint>
#include <cstdarg>
#include <vector>
#include <thread>
#include <algorithm>
#include <functional>
#include "../../include/sddmm.h"

struct sddmm_coo {
    int64_t n_rows = 0, n_cols = 0, nnz = 0;
    std::vector<int32_t> rows, cols;
    std::vector<float> vals;
    int sorted = 0;  // 1: (row, col)-sorted.  Set by whatever creates or reorders the matrix, never lazily.
};

// Tile-order view of a sorted matrix: tiles ascending, rows ascending inside a
// tile, columns ascending inside a row (the order rewrite_matrix_1D produces,
// HiPC18/src/util.h:267-343), stored compactly.
struct sddmm_tiling {
    int32_t tile_x = 0, tile_y = 0, n_tiles = 0;
    int64_t nnz = 0, n_rows = 0, n_cols = 0;
    std::vector<int32_t> tile_ptr;    // [n_tiles+1] offsets in tile order
    std::vector<int32_t> tiled_ind;   // [nnz] original position of each tile-order nonzero
    std::vector<int64_t> active_ptr;  // [n_tiles+1] offsets into active_row/active_end
    std::vector<int32_t> active_row;  // global row id of each (tile, active row)
    std::vector<int32_t> active_end;  // tile-order end offset of that row's run
    std::vector<int64_t> block_ptr;   // [n_tiles+1] offsets into block_end
    std::vector<int32_t> block_end;   // tile-order end offset after every tile_y active rows
    int32_t max_active_rows = 0;
};

namespace sddmm {

void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

int hw_threads();

// Runs f(begin, end, thread_index) over [0, n) split into at most hw_threads()
// contiguous ranges (one range if n < grain).
void parallel_ranges(int64_t n, int64_t grain,
                     const std::function<void(int64_t, int64_t, int)> &f, int *n_used = nullptr);

// Runs f(begin, end, thread_index) over [0, n) in chunks of `chunk` that the threads
// take in turn from a shared counter (for work of uneven cost per index).
void parallel_dynamic(int64_t n, int64_t chunk, const std::function<void(int64_t, int64_t, int)> &f);

// out[p] = softmax over the entries of p's row of x (out may be x), on `stream` (a hipStream_t).  d_ws: device memory of
// row_softmax_workspace_bytes(nnz) bytes for the pass's records, nnz the number of entries (d_row_ptr[n_rows]); null: the
// library's own per-device arrays, which calls that overlap in time would share.
int launch_row_softmax(int64_t n_rows, const int32_t *d_row_ptr, const float *d_x, float *d_out, void *stream, void *d_ws, int64_t nnz);
int64_t row_softmax_workspace_bytes(int64_t nnz);

bool check_sorted(const sddmm_coo &S);
// CSR row pointers of a sorted matrix (n_rows+1 entries).
void build_row_ptr(const sddmm_coo &S, std::vector<int32_t> &row_ptr);

// The tiling pass proper, on raw CSR arrays (host).
int build_tiling(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                 const int32_t *col_ind, int32_t tile_x, int32_t tile_y, sddmm_tiling &T,
                 const int32_t *row_list, int64_t n_list);

// The dense core of a sorted matrix, cut out for the dense-block kernel: blocks of `tile`
// rows of similar length x `tile` columns that at least the threshold share of those rows
// have, each listed with its nonzeros; everything else is left as a CSR remainder with a map
// back to the positions in the original S.
struct DenseBlocks {
    int32_t tile = 0;
    std::vector<int32_t> row_ids;   // [n_row_blocks * tile] rows in rank order (padded with row_ids[0])
    std::vector<int32_t> col_ids;   // [n_tiles * tile] columns of each block, ascending (a short group repeats its last one)
    std::vector<int32_t> tile_rb;   // [n_tiles] row block of each block; blocks of a row block are consecutive
    std::vector<int32_t> tile_ptr;  // [n_tiles + 1]
    std::vector<int32_t> nz_p;      // [n_dense] position in the original S
    std::vector<uint16_t> nz_rc;    // [n_dense] (row in block << 8) | column in block
    int64_t n_dense = 0;
    // the remainder, rows as in S
    std::vector<int32_t> rem_row_ptr;  // [n_rows + 1]
    std::vector<int32_t> rem_col;      // [nnz - n_dense]
    std::vector<int32_t> rem_orig;     // [nnz - n_dense] position in the original S
};
// threshold: least share of a block's rows that must have a column for it to be dense there.  Leaves D.n_dense == 0
// (and the remainder arrays empty) when fewer than min_dense nonzeros would qualify.
int find_dense_blocks(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr, const int32_t *col_ind,
                      int32_t tile, double threshold, int64_t min_dense, DenseBlocks &D);

}  // namespace sddmm
