// The tiling / reorder pass: cuts a (row, col)-sorted matrix into column tiles
// of tile_x columns and, inside each tile, into panels of tile_y active rows.
// It produces the order rewrite_matrix_1D produces (HiPC18/src/util.h:267-343:
// tiles ascending, rows ascending inside a tile, columns ascending inside a
// row) as a permutation of the original positions; nonzeros themselves stay
// where they are.  Unlike the reference (serial, O(n_tiles * n_rows + nnz) time
// and an n_rows * n_tiles table, util.h:62) this runs on all host threads in
// O(nnz + threads * n_tiles) time and O(nnz + segments) space.
#include "internal.hpp"
#include <cstring>

namespace sddmm {

int build_tiling(int64_t n_rows, int64_t n_cols, int64_t nnz_all, const int32_t *row_ptr,
                 const int32_t *col_ind, int32_t tile_x, int32_t tile_y, sddmm_tiling &T,
                 const int32_t *row_list, int64_t n_list)
{
    // row_list != null: only those rows (ascending) take part; offsets then count their nonzeros only
    const int64_t n_it = row_list ? n_list : n_rows;
    auto row_of = [&](int64_t i) -> int64_t { return row_list ? row_list[i] : i; };
    int64_t nnz = nnz_all;
    if (row_list) {
        nnz = 0;
        for (int64_t i = 0; i < n_list; ++i) nnz += row_ptr[row_list[i] + 1] - row_ptr[row_list[i]];
    }
    if (tile_x < 1 || tile_y < 1) return fail(SDDMM_ERR_ARG, "tiling: tile sizes must be >= 1");
    const int64_t n_tiles = std::max<int64_t>(1, (n_cols + tile_x - 1) / tile_x);
    if (n_tiles >= INT32_MAX) return fail(SDDMM_ERR_RANGE, "tiling: too many column tiles");
    T.tile_x = tile_x; T.tile_y = tile_y; T.n_tiles = (int32_t)n_tiles;
    T.nnz = nnz; T.n_rows = n_rows; T.n_cols = n_cols;

    // Threads own contiguous row ranges balanced by nonzeros.
    int nt = (int)std::max<int64_t>(1, std::min<int64_t>(hw_threads(), nnz / (1 << 15) + 1));
    std::vector<int64_t> rb((size_t)nt + 1);
    rb[0] = 0; rb[nt] = n_it;
    if (row_list) {
        int64_t acc = 0;
        int t = 1;
        for (int64_t i = 0; i < n_list && t < nt; ++i) {
            acc += row_ptr[row_list[i] + 1] - row_ptr[row_list[i]];
            while (t < nt && acc >= nnz * t / nt) rb[t++] = i + 1;
        }
        for (; t < nt; ++t) rb[t] = n_list;
    } else {
        for (int t = 1; t < nt; ++t) {
            int64_t target = nnz * t / nt;
            rb[t] = std::lower_bound(row_ptr, row_ptr + n_rows + 1, (int32_t)target) - row_ptr;
            rb[t] = std::min<int64_t>(std::max(rb[t], rb[t - 1]), n_rows);
        }
    }
    // pass 1: per thread, nonzeros and (row, tile) runs per tile
    std::vector<std::vector<int64_t>> cnt_nnz(nt, std::vector<int64_t>((size_t)n_tiles, 0));
    std::vector<std::vector<int64_t>> cnt_seg(nt, std::vector<int64_t>((size_t)n_tiles, 0));
    auto run_threads = [&](const std::function<void(int)> &f) {
        if (nt == 1) { f(0); return; }
        std::vector<std::thread> th;
        for (int t = 0; t < nt; ++t) th.emplace_back(f, t);
        for (auto &x : th) x.join();
    };
    run_threads([&](int t) {
        auto &cn = cnt_nnz[t];
        auto &cs = cnt_seg[t];
        for (int64_t ri = rb[t]; ri < rb[t + 1]; ++ri) {
            const int64_t r = row_of(ri);
            int64_t i = row_ptr[r], e = row_ptr[r + 1];
            while (i < e) {
                int64_t tile = col_ind[i] / tile_x;
                int64_t lim = (tile + 1) * (int64_t)tile_x;
                int64_t j = i + 1;
                while (j < e && col_ind[j] < lim) ++j;
                cn[tile] += j - i;
                cs[tile] += 1;
                i = j;
            }
        }
    });
    // offsets: tile-major, then thread (= row) order
    T.tile_ptr.assign((size_t)n_tiles + 1, 0);
    T.active_ptr.assign((size_t)n_tiles + 1, 0);
    std::vector<std::vector<int64_t>> off_nnz(nt, std::vector<int64_t>((size_t)n_tiles));
    std::vector<std::vector<int64_t>> off_seg(nt, std::vector<int64_t>((size_t)n_tiles));
    int64_t acc_n = 0, acc_s = 0;
    for (int64_t j = 0; j < n_tiles; ++j) {
        T.tile_ptr[j] = (int32_t)acc_n;
        T.active_ptr[j] = acc_s;
        for (int t = 0; t < nt; ++t) {
            off_nnz[t][j] = acc_n; acc_n += cnt_nnz[t][j];
            off_seg[t][j] = acc_s; acc_s += cnt_seg[t][j];
        }
    }
    T.tile_ptr[n_tiles] = (int32_t)acc_n;
    T.active_ptr[n_tiles] = acc_s;
    try {
        T.tiled_ind.resize((size_t)nnz);
        T.active_row.resize((size_t)acc_s);
        T.active_end.resize((size_t)acc_s);
    } catch (const std::exception &) {
        return fail(SDDMM_ERR_NOMEM, "tiling: out of memory (%lld nonzeros, %lld row runs)", (long long)nnz, (long long)acc_s);
    }
    // pass 2: write the permutation and the active-row lists
    run_threads([&](int t) {
        auto &on = off_nnz[t];
        auto &os = off_seg[t];
        for (int64_t ri = rb[t]; ri < rb[t + 1]; ++ri) {
            const int64_t r = row_of(ri);
            int64_t i = row_ptr[r], e = row_ptr[r + 1];
            while (i < e) {
                int64_t tile = col_ind[i] / tile_x;
                int64_t lim = (tile + 1) * (int64_t)tile_x;
                int64_t d = on[tile];
                int64_t j = i;
                while (j < e && col_ind[j] < lim) T.tiled_ind[d++] = (int32_t)j++;
                on[tile] = d;
                T.active_row[os[tile]] = (int32_t)r;
                T.active_end[os[tile]] = (int32_t)d;
                os[tile]++;
                i = j;
            }
        }
    });
    // panels: a boundary after every tile_y active rows of a tile, and at its end
    T.block_ptr.assign((size_t)n_tiles + 1, 0);
    int64_t nb = 0;
    int64_t max_act = 0;
    for (int64_t j = 0; j < n_tiles; ++j) {
        T.block_ptr[j] = nb;
        int64_t na = T.active_ptr[j + 1] - T.active_ptr[j];
        max_act = std::max(max_act, na);
        nb += (na + tile_y - 1) / tile_y;
    }
    T.block_ptr[n_tiles] = nb;
    T.max_active_rows = (int32_t)max_act;
    T.block_end.resize((size_t)nb);
    parallel_ranges(n_tiles, 64, [&](int64_t jb, int64_t je, int) {
        for (int64_t j = jb; j < je; ++j) {
            int64_t a0 = T.active_ptr[j], a1 = T.active_ptr[j + 1];
            int64_t b = T.block_ptr[j];
            for (int64_t a = a0; a < a1; a += tile_y) {
                int64_t last = std::min<int64_t>(a + tile_y, a1) - 1;
                T.block_end[b++] = T.active_end[last];
            }
        }
    });
    return SDDMM_OK;
}

}  // namespace sddmm

using namespace sddmm;

extern "C" int sddmm_tiling_create(const sddmm_coo *S, int32_t tile_size_x, int32_t tile_size_y,
                                   sddmm_tiling **out)
{
    if (!S || !out) return fail(SDDMM_ERR_ARG, "sddmm_tiling_create: NULL argument");
    *out = nullptr;
    if (S->sorted != 1) return fail(SDDMM_ERR_UNSORTED, "sddmm_tiling_create: matrix is not (row, col)-sorted");
    sddmm_tiling *T = new (std::nothrow) sddmm_tiling;
    if (!T) return fail(SDDMM_ERR_NOMEM, "sddmm_tiling_create: out of memory");
    int rc;
    try {
        std::vector<int32_t> rp;
        build_row_ptr(*S, rp);
        rc = build_tiling(S->n_rows, S->n_cols, S->nnz, rp.data(), S->cols.data(), tile_size_x, tile_size_y, *T, nullptr, 0);
    } catch (const std::exception &) {
        rc = fail(SDDMM_ERR_NOMEM, "sddmm_tiling_create: out of memory");
    }
    if (rc) { delete T; return rc; }
    *out = T;
    return SDDMM_OK;
}

extern "C" int sddmm_tiling_get(const sddmm_tiling *T, sddmm_tiling_view *v)
{
    if (!T || !v) return fail(SDDMM_ERR_ARG, "sddmm_tiling_get: NULL argument");
    v->tile_size_x = T->tile_x; v->tile_size_y = T->tile_y; v->n_col_tiles = T->n_tiles;
    v->nnz = T->nnz;
    v->max_active_rows = T->max_active_rows;
    v->tile_ptr = T->tile_ptr.data();
    v->tiled_ind = T->tiled_ind.data();
    v->active_ptr = T->active_ptr.data();
    v->active_row = T->active_row.data();
    v->active_end = T->active_end.data();
    v->block_ptr = T->block_ptr.data();
    v->block_end = T->block_end.data();
    return SDDMM_OK;
}

extern "C" void sddmm_tiling_destroy(sddmm_tiling *T) { delete T; }
