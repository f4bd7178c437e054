// Finds the dense core of a sorted sparse matrix for the dense-block kernel.
//
// Power-law matrices (ratings, bags of words) have heavy rows and popular
// columns whose intersections are mostly filled.  Rows are ranked by length
// (only those long enough to take part in a block of the wanted density at all)
// and cut into row blocks of `tile` rows of similar length.  For each row block
// the columns that at least `threshold` of its rows have are its dense columns;
// in ascending column order they are cut into groups of `tile`, and each (row
// block, column group) pair is a block for the dense kernel, filled to the
// threshold or better by construction.  Keeping the dense columns of a block in
// column order keeps a row's nonzeros of that block next to each other in the
// sorted S, so their results are stored to neighbouring addresses.  What is
// left stays a CSR matrix (rows and in-row order as in S) with a map to the
// original positions, for the gathering kernels.  The idea of splitting a
// matrix into a dense and a sparse part by segment occupancy is the reference's
// experiment other_ideas/our_work/sparse_dense_split/util.h:211-274; the
// selection here works per column inside blocks of degree-ranked rows instead
// of per-row half tiles.  All passes are O(nnz) and run on all host threads.
#include "internal.hpp"
#include <atomic>
#include <cmath>

namespace sddmm {

namespace {

// ids with key >= kmin in descending key order (ties: ascending id); counting sort
void rank_desc(const std::vector<int32_t> &key, int32_t kmin, std::vector<int32_t> &order)
{
    int32_t kmax = 0;
    for (int32_t k : key) kmax = std::max(kmax, k);
    order.clear();
    if (kmax < kmin) return;
    std::vector<int64_t> start((size_t)(kmax - kmin) + 2, 0);
    for (int32_t k : key)
        if (k >= kmin) ++start[(size_t)(kmax - k) + 1];
    for (size_t i = 1; i < start.size(); ++i) start[i] += start[i - 1];
    order.resize((size_t)start.back());
    for (size_t id = 0; id < key.size(); ++id)
        if (key[id] >= kmin) order[(size_t)start[(size_t)(kmax - key[id])]++] = (int32_t)id;
}

}  // namespace

int find_dense_blocks(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr, const int32_t *col_ind,
                      int32_t tile, double threshold, int64_t min_dense, DenseBlocks &D)
{
    D = DenseBlocks{};
    D.tile = tile;
    if (tile < 2 || tile > 256 || threshold <= 0.0 || nnz < (int64_t)tile * tile / 2) return SDDMM_OK;
    // a column is dense in a row block when this many of the block's rows have it
    const int32_t need = (int32_t)std::max<int64_t>(1, (int64_t)std::ceil(threshold * tile));
    // a column group may be filled up with repeated columns when at least this many are real
    const int32_t min_group = tile - tile / 4;

    // rows that can be part of a dense block at all (a block has `tile` columns, `need` of which
    // an average row of it must have), longest first
    std::vector<int32_t> deg((size_t)n_rows);
    parallel_ranges(n_rows, 1 << 14, [&](int64_t b, int64_t e, int) {
        for (int64_t r = b; r < e; ++r) deg[(size_t)r] = row_ptr[r + 1] - row_ptr[r];
    });
    std::vector<int32_t> rows_c;
    rank_desc(deg, need, rows_c);
    if ((int64_t)rows_c.size() < tile / 2) return SDDMM_OK;
    const int64_t n_rb = ((int64_t)rows_c.size() + tile - 1) / tile;
    if (n_rb * tile >= INT32_MAX) return SDDMM_OK;

    // pass 1, one row block at a time: its dense columns, cut into groups; nonzeros per group and
    // how many nonzeros each row keeps for the remainder
    struct BlockSel { std::vector<int32_t> cols; std::vector<int32_t> group_nnz; };  // cols: groups x tile, ascending inside a group
    std::vector<BlockSel> selb((size_t)n_rb);
    std::vector<int32_t> keep(deg);
    const int nt = hw_threads();
    // (every thread keeps two words per column: a wide matrix on a host with many threads would spend
    // gigabytes here to learn that it has no dense core -- such a matrix goes without dense blocks)
    if ((int64_t)n_cols * 8 * nt > ((int64_t)1 << 30)) return SDDMM_OK;
    std::vector<std::vector<int32_t>> cnt_t((size_t)nt), slot_t((size_t)nt);
    parallel_dynamic(n_rb, 1, [&](int64_t b, int64_t e, int t) {
        std::vector<int32_t> &cnt = cnt_t[(size_t)t], &slot = slot_t[(size_t)t];
        if (cnt.empty()) { cnt.assign((size_t)n_cols, 0); slot.assign((size_t)n_cols, -1); }
        std::vector<int32_t> touched, pick;
        for (int64_t rb = b; rb < e; ++rb) {
            const int64_t i0 = rb * tile, i1 = std::min<int64_t>(i0 + tile, (int64_t)rows_c.size());
            for (int64_t i = i0; i < i1; ++i) {
                const int32_t r = rows_c[(size_t)i];
                for (int32_t p = row_ptr[r]; p < row_ptr[r + 1]; ++p)
                    if (cnt[(size_t)col_ind[p]]++ == 0) touched.push_back(col_ind[p]);
            }
            pick.clear();
            for (int32_t c : touched)
                if (cnt[(size_t)c] >= need) pick.push_back(c);
            // whole groups only: the columns with the fewest nonzeros are left out (or, when nearly a
            // whole group is left over, it is kept and filled up)
            int64_t groups = (int64_t)pick.size() / tile;
            const int64_t rest = (int64_t)pick.size() % tile;
            if (rest >= min_group) ++groups;
            else if (rest) {
                std::nth_element(pick.begin(), pick.begin() + (pick.size() - rest), pick.end(),
                                 [&](int32_t x, int32_t y) { return cnt[(size_t)x] != cnt[(size_t)y] ? cnt[(size_t)x] > cnt[(size_t)y] : x < y; });
                pick.resize(pick.size() - (size_t)rest);
            }
            for (int32_t c : touched) cnt[(size_t)c] = 0;
            touched.clear();
            if (groups == 0) continue;
            std::sort(pick.begin(), pick.end());
            BlockSel &bs = selb[(size_t)rb];
            bs.cols.assign((size_t)(groups * tile), pick.back());  // a filled-up group repeats its last column
            std::copy(pick.begin(), pick.end(), bs.cols.begin());
            bs.group_nnz.assign((size_t)groups, 0);
            for (size_t k = 0; k < pick.size(); ++k) slot[(size_t)pick[k]] = (int32_t)k;
            for (int64_t i = i0; i < i1; ++i) {
                const int32_t r = rows_c[(size_t)i];
                int32_t taken = 0;
                for (int32_t p = row_ptr[r]; p < row_ptr[r + 1]; ++p) {
                    const int32_t k = slot[(size_t)col_ind[p]];
                    if (k >= 0) { ++bs.group_nnz[(size_t)(k / tile)]; ++taken; }
                }
                keep[(size_t)r] -= taken;
            }
            for (int32_t c : pick) slot[(size_t)c] = -1;
        }
    });
    int64_t n_tiles = 0, n_dense = 0;
    std::vector<int64_t> rb_first((size_t)n_rb + 1, 0);
    for (int64_t rb = 0; rb < n_rb; ++rb) {
        rb_first[(size_t)rb] = n_tiles;
        n_tiles += (int64_t)selb[(size_t)rb].group_nnz.size();
        for (int32_t g : selb[(size_t)rb].group_nnz) n_dense += g;
    }
    rb_first[(size_t)n_rb] = n_tiles;
    if (n_tiles == 0 || n_dense < min_dense || n_dense >= INT32_MAX || n_tiles * tile >= INT32_MAX) return SDDMM_OK;

    D.tile_rb.resize((size_t)n_tiles); D.tile_ptr.assign((size_t)n_tiles + 1, 0);
    D.col_ids.resize((size_t)(n_tiles * tile));
    for (int64_t rb = 0; rb < n_rb; ++rb) {
        const BlockSel &bs = selb[(size_t)rb];
        const int64_t k0 = rb_first[(size_t)rb];
        for (size_t g = 0; g < bs.group_nnz.size(); ++g) {
            D.tile_rb[(size_t)k0 + g] = (int32_t)rb;
            D.tile_ptr[(size_t)k0 + g + 1] = bs.group_nnz[g];
        }
        std::copy(bs.cols.begin(), bs.cols.end(), D.col_ids.begin() + (size_t)(k0 * tile));
    }
    for (int64_t k = 0; k < n_tiles; ++k) D.tile_ptr[(size_t)k + 1] += D.tile_ptr[(size_t)k];
    D.rem_row_ptr.assign((size_t)n_rows + 1, 0);
    for (int64_t r = 0; r < n_rows; ++r) D.rem_row_ptr[(size_t)r + 1] = D.rem_row_ptr[(size_t)r] + keep[(size_t)r];
    const int64_t n_rem = D.rem_row_ptr[(size_t)n_rows];
    if (n_rem + n_dense != nnz) return fail(SDDMM_ERR_ARG, "dense blocks: %lld + %lld nonzeros of %lld accounted for",
                                            (long long)n_dense, (long long)n_rem, (long long)nnz);

    // pass 2: the blocks' nonzero lists (rows in rank order, positions ascending inside a row) and
    // the remainder of the ranked rows
    D.nz_p.resize((size_t)n_dense); D.nz_rc.resize((size_t)n_dense);
    D.rem_col.resize((size_t)n_rem); D.rem_orig.resize((size_t)n_rem);
    std::vector<uint8_t> ranked((size_t)n_rows, 0);
    for (int32_t r : rows_c) ranked[(size_t)r] = 1;
    parallel_dynamic(n_rb, 1, [&](int64_t b, int64_t e, int t) {
        std::vector<int32_t> &slot = slot_t[(size_t)t];
        if (slot.empty()) slot.assign((size_t)n_cols, -1);
        std::vector<int32_t> cursor;
        for (int64_t rb = b; rb < e; ++rb) {
            const BlockSel &bs = selb[(size_t)rb];
            const int64_t k0 = rb_first[(size_t)rb], groups = (int64_t)bs.group_nnz.size();
            cursor.assign(D.tile_ptr.begin() + k0, D.tile_ptr.begin() + k0 + groups);
            // (a filled-up group repeats its last column: the first of the equal entries keeps the slot)
            for (size_t k = bs.cols.size(); k-- > 0;) slot[(size_t)bs.cols[k]] = (int32_t)k;
            const int64_t i0 = rb * tile, i1 = std::min<int64_t>(i0 + tile, (int64_t)rows_c.size());
            for (int64_t i = i0; i < i1; ++i) {
                const int32_t r = rows_c[(size_t)i];
                int64_t d = D.rem_row_ptr[(size_t)r];
                for (int32_t p = row_ptr[r]; p < row_ptr[r + 1]; ++p) {
                    const int32_t k = slot[(size_t)col_ind[p]];
                    if (k >= 0) {
                        const int32_t at = cursor[(size_t)(k / tile)]++;
                        D.nz_p[(size_t)at] = p;
                        D.nz_rc[(size_t)at] = (uint16_t)(((i - i0) << 8) | (k % tile));
                    } else {
                        D.rem_col[(size_t)d] = col_ind[p];
                        D.rem_orig[(size_t)d] = p;
                        ++d;
                    }
                }
            }
            for (int32_t c : bs.cols) slot[(size_t)c] = -1;
        }
    });
    // rows outside the ranking keep all their nonzeros
    parallel_dynamic(n_rows, 4096, [&](int64_t b, int64_t e, int) {
        for (int64_t r = b; r < e; ++r) {
            if (ranked[(size_t)r]) continue;
            int64_t d = D.rem_row_ptr[(size_t)r];
            for (int32_t p = row_ptr[r]; p < row_ptr[r + 1]; ++p, ++d) {
                D.rem_col[(size_t)d] = col_ind[p];
                D.rem_orig[(size_t)d] = p;
            }
        }
    });

    D.row_ids.assign((size_t)(n_rb * tile), rows_c[0]);
    std::copy(rows_c.begin(), rows_c.end(), D.row_ids.begin());
    D.n_dense = n_dense;
    return SDDMM_OK;
}

}  // namespace sddmm
