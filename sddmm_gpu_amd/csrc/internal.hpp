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
    int sorted = -1;  // -1 unknown, 0 no, 1 (row, col)-sorted
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

bool check_sorted(const sddmm_coo &S);
// CSR row pointers of a sorted matrix (n_rows+1 entries).
void build_row_ptr(const sddmm_coo &S, std::vector<int32_t> &row_ptr);

// The tiling pass proper, on raw CSR arrays (host).
int build_tiling(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                 const int32_t *col_ind, int32_t tile_x, int32_t tile_y, sddmm_tiling &T,
                 const int32_t *row_list, int64_t n_list);

}  // namespace sddmm
