// Argument blocks and lookup functions shared by the plan builder (planner.hip, planner_tile.hip), the launch code (engine.hip)
// and the kernel translation units.
#pragma once
#include <cstdint>
#include <hip/hip_vector_types.h>

namespace sddmm {

struct WorkItem {
    int32_t begin, end;   // stream positions
    int32_t batch_base;   // index of the item's first batch in batch_seg / batch_mask (tile kernel: in btype)
    int32_t tile;         // column tile staged in LDS (-1: none)
};

struct KArgs {
    const int32_t *col_ind;    // [nnz] sorted order
    const float *val;          // [nnz] or null (no scaling)
    const float *W, *H;
    float *out;
    const int32_t *perm;       // stream position -> sorted position, null = identity
    const int32_t *scol;       // column indices in stream order, or null (use col_ind[perm])
    const float *sval;         // values in stream order, or null (use val[perm])
    const int32_t *seg_row;    // segment -> global row, null = identity
    const int32_t *batch_seg;  // per batch: segment of its first nonzero
    const uint64_t *batch_mask;  // per batch: bit L (L >= 1) set if lane L starts a new segment
    const WorkItem *items;     // null: fixed chunks of `chunk` nonzeros over [0, nnz)
    int32_t n_items;
    int32_t nnz;
    int32_t chunk;
    int32_t K;
    int32_t tile_x;
    int32_t n_cols;
    int32_t generic_perm;
    int32_t residual;          // 0: out = val * dot;  1: out = val - dot
    // Plan-free form (batch_seg and batch_mask are null then): batch_row[b] is the row of stream
    // position 64*b, and every lane finds its own row by a search of row_ptr between the
    // rows of two consecutive batches.
    const int32_t *row_ptr;    // [n_rows+1]
    const int32_t *batch_row;  // [ceil(nnz/64)]
    int32_t n_rows;
};

constexpr int kRowGatherBlock = 256;   // 4 waves
constexpr int kRowGatherBatchesPerWave = 8;
constexpr int kLdsBlock = 1024;        // 16 waves, one workgroup per CU
constexpr int kLdsMaxBytes = 160 * 1024;

struct Variant {
    int G, KPL;   // lanes per nonzero, float4 slots per lane
    bool exact;   // K == 4*G*KPL
};
using KernelFn = void (*)(const KArgs);

// Tile kernel: padded tile-order stream, H tiles in LDS.
struct TileArgs {
    // (a padding position repeats the last nonzero of its run in perm, scol and sval)
    const int32_t *perm;   // stream position -> sorted position
    const int32_t *scol;   // per stream position: byte offset of the column's H row inside the LDS tile;
                           // gather form: index of the H row's first float4, column * K/4
    const int32_t *grow;   // per group of G consecutive stream positions: index of the W row's first float4, row * K/4
    const float *sval;     // values in stream order or null
    // Compact form (LDS tiles of a K slice of at most 64 elements, where the kernel is bound by
    // the bytes it streams): scol16 replaces scol with the column's index inside the tile,
    // pbase replaces perm with one word per group of G positions -- the sorted position of
    // the group's first nonzero; its nonzeros are consecutive there -- and grow carries the
    // group's number of nonzeros minus one in its low bits (rows are K/4 >= 8 float4 long).
    const uint16_t *scol16;
    const int32_t *pbase;
    // One bit per batch of 64 positions, counted from WorkItem::batch_base inside an item: set for a
    // "short" batch, whose groups hold at most G/2 nonzeros each, in positions 0 .. G/2-1 and once
    // more in G/2 .. G-1 (see tile_variant_shorts).  Null: no short batches.
    const uint32_t *btype;
    const float *val;      // values in sorted order or null
    const float *W, *H;
    float *out;
    float *part;               // partial results in stream order between the K slices of a sliced launch (else null)
    int32_t to_part;           // sliced launch: this slice stores to part (every slice but the last)
    float *sink;               // gather form: 256 x 64 floats that take the results of flagged padding positions
    const int32_t *unit_ptr;   // [n_units+1] first stream position of each (row panel, column tile) unit
    const int32_t *unit_tile;  // [n_units] the unit's column tile
    int32_t n_units;
    const WorkItem *items;     // non-null: workgroup b works on items b, b + grid, ... (each inside one tile)
    int32_t n_items;
    int32_t tile_x, n_cols;
    int32_t K;           // row length of W and H
    int32_t k_off;       // first K element covered by this launch (the kernel's own width is 4*G*KPL)
    int32_t n_slices;    // the all-slices-in-one-launch form: K slices walked inside the launch, from k_off on
    // Matrix-core share of a launch (kernel variants with NWM > 0; mf_groups == 0: none).  The heaviest
    // rows, in groups of 32, are multiplied as whole 32 x 32 blocks against blocks of 32 consecutive
    // columns by the last NWM waves of every workgroup, from operands packed by sddmm_mf_pack_kernel:
    //   mf_hp[(cb * 32 + p) * 32 + j] = float4 p of the K slice of H row 32 cb + j (zero beyond n_cols)
    //   mf_wp[(g * 32 + p) * 32 + i]  = float4 p of the K slice of W row mf_rows[32 g + i]
    // (an MFMA operand load of one wave is then 1 KB of consecutive addresses).  Groups [die * G, (die + 1) * G),
    // G = mf_groups / 8, belong to the workgroups of that die (workgroup b runs on die b % 8); a die's
    // (group, column block) pairs are numbered column block by column block, q = cb * G + (g - die * G), and
    // mf_rowinfo[(die * G * mf_n_cb + q) * 32 + i] = {bit j set: S has (row i of the group, column 32 cb + j);
    // sorted position of the row's first nonzero in that block}: the nonzero of bit j sits at that
    // position plus the number of set bits below j.
    const float4 *mf_hp, *mf_wp;
    const uint2 *mf_rowinfo;
    const int32_t *mf_rows;   // [32 * mf_groups] rows of the groups (a short last group repeats a row, with empty masks)
    int32_t mf_groups, mf_n_cb;
    int32_t nnz;              // of S (bound for value reads)
    int32_t tile_bytes;       // bytes of the H tile in LDS (the matrix-core waves' own LDS follows it)
};
struct TileVariant {
    int G, KPL;  // lanes per nonzero, float4 per lane; K == 4*G*KPL
};
using TileFn = void (*)(const TileArgs);
// Variants that can skip half the steps of a batch marked short in TileArgs::btype.
constexpr bool tile_variant_shorts(int G, int KPL, bool gather)
{
    return !gather && G == 8 && (G * KPL) % 16 == 0 && G * KPL > 16;
}
// want_g > 0: that group size or nothing; 0: the preferred one for K
TileVariant pick_tile_variant(int K, int want_g);
// vmode: 0 = values in stream order (sval), 1 = values in sorted order (val), 2 = no values
// gather: H rows from global memory, 4 waves per workgroup (otherwise H tiles in LDS, nwaves = 16 or 12 waves)
// slice: 0 the launch covers all of K, 1 first of several K slices, 2 a later one (see the kernel template)
TileFn tile_kernel(const TileVariant &v, int vmode, bool gather, int slice, int nwaves);
// The variant with a matrix-core share (TileArgs::mf_*): groups of 8 lanes on rows of 128 elements, all of K
// in one launch, nw vector waves + nwm matrix-core waves per workgroup ((12, 4), (8, 8) or (8, 4)).
TileFn tile_kernel_mf(int vmode, int nw, int nwm);
constexpr int kMfLdsExtra = 64;        // bytes of LDS behind the H tile for the vector waves' barrier counter ...
constexpr int kMfLdsPerWave = 512;     // ... and for each matrix-core wave's row masks
// packs the operands of the matrix-core share (a.mf_hp from a.H, a.mf_wp from a.W through a.mf_rows) on `stream`
void launch_mf_pack(const TileArgs &a, void *stream);

// Sparse-times-dense product Y = X H on a tile launch's column tiles (kernels_spmm.hip).  The rows of the
// launch are walked as (row, tile) runs; eight runs of about equal length make a bundle, walked side by side
// by the eight lane groups of a wave.
struct SpmmArgs {
    const WorkItem *items;     // per (row block, tile) item: [begin, end) = its bundles, tile = its column tile
    int32_t n_items;
    const int32_t *b_off;      // [n_bundles + 1] first round of each bundle (a round: 8 steps x 8 groups)
    const int32_t *b_p0;       // [8 n_bundles] sorted position of each group's first nonzero (its run is consecutive there)
    const int32_t *b_len;      // [8 n_bundles] nonzeros of each group's run (0: no run)
    const uint16_t *cols;      // [rounds][8 groups][8 steps] column inside the tile (beyond the run: its last column again)
    const float *x;            // [nnz] sorted order
    const float *H;
    float *part;               // [8 n_bundles][k slice] partial rows, one per run
    float *Y;
    const int32_t *row_part_ptr, *part_slot, *sum_rows;  // rows with runs: their partial rows (CSR-like) and their numbers
    int64_t n_sum_rows;
    const int32_t *gather_rows;  // the launch's other rows (gathered from global memory; rows without entries included)
    int64_t n_gather_rows;
    const int32_t *row_ptr, *col_ind;
    int32_t tile_x, n_cols, K, k_off;
};
bool spmm_tile_supported(int k_slice);
int spmm_tile_set_lds(int k_slice, int nwaves, int lds_bytes);  // 0 ok, 1 no such variant, 2 HIP error
void launch_spmm_slice(const SpmmArgs &a, int k_slice, int nwaves, int grid, int lds_bytes, void *stream);

// dst[i] = perm[i] >= 0 ? src[perm[i]] : 0 for i < n, on `stream` (a hipStream_t)
void launch_gather_values(const int32_t *perm, const float *src, float *dst, int64_t n, void *stream);

// Panel kernel: rows of W resident in VGPRs, column tiles of H in LDS.
struct PanelArgs {
    const int32_t *row_ptr;   // [n_rows+1]
    const int32_t *col_ind;   // [nnz] sorted order
    const float *val;         // [nnz] or null (no scaling)
    const float *W, *H;
    float *out;
    const int32_t *slot_row;  // [n_panels][S][NWAVES][8] row of each (slot, wave, group); -1 = none
    const int32_t *panel_tiles;  // [n_panels][2] first and last column tile the panel touches
    int32_t n_panels, tile_x, n_cols;
    int32_t K;                // row length of W and H
    int32_t k_off;            // first K element covered by this pass
    int32_t accumulate;       // add to out instead of overwriting it
    int32_t residual;         // 0: out = val * dot;  1: out = val - dot (later K slices: out -= dot)
};
struct PanelVariant {
    int KPL, S, NWAVES;       // float4 per lane (K slice = 32*KPL), row slots per 8-lane group, waves per workgroup
};
using PanelFn = void (*)(const PanelArgs);
PanelVariant pick_panel_variant(int k_slice);
PanelFn panel_kernel(const PanelVariant &v);

// Dense-block kernel: blocks of kDenseTile listed rows x kDenseTile listed columns computed
// whole on the matrix cores; the block's nonzeros pick their results.
constexpr int kDenseTile = 128;
struct DenseArgs {
    // Workgroup b takes slots b, b + grid, ...; a workgroup's filled slots come first.
    const int32_t *slot_rows;  // [n_slots][kDenseTile] rows of the slot's block (a short row block padded with a valid row)
    const int32_t *slot_cols;  // [n_slots][kDenseTile] its columns
    const int2 *slot_range;    // [n_slots] the block's nonzeros in nz_*: [x, y); x == y: empty slot
    const int32_t *nz_p;      // sorted position of each nonzero
    const uint16_t *nz_rc;    // (row inside the block << 8) | column inside the block
    const float *nz_val;      // values in list order or null
    const float *val;         // values in sorted order or null (both null: no scaling)
    const float *W, *H;
    float *out;
    int32_t n_slots;
    int32_t K;                // row length of W and H, a multiple of 32
    int32_t residual;         // 0: out = val * dot;  1: out = val - dot
};
using DenseFn = void (*)(const DenseArgs);
DenseFn dense_kernel();

// lanes per nonzero and float4 slots per lane for a given K (K % 4 == 0); G == 0: none
Variant pick_variant(int K, bool lds_tile);
KernelFn stream_kernel(const Variant &v, bool lds_tile);
KernelFn generic_kernel();

}  // namespace sddmm
