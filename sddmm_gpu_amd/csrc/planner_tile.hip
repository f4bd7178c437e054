// The tile launch of the SDDMM planner for gfx950 (MI355X): stream layout, padding, short batches,
// work assignment across dies, the opt-in matrix-core share and the SpMM stream on the same tiles.
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstring>
#include <new>
#include <unistd.h>
#include "plan.hpp"

namespace sddmm {

// Tile launch: the rows' nonzeros in tile order (tiles of x columns), every
// (row, tile) run padded to a multiple of G stream positions.
int add_tile(Ctx &c, const std::vector<int32_t> &rows_in, int32_t x, int32_t panel_rows, int want_g, int ks,
             sddmm_plan_info *I, bool gather, bool x_explicit)
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

}  // namespace sddmm
