/*
 * sddmm.h -- C ABI of the MI355X (gfx950) SDDMM engine.
 *
 *   out[p] = S.val[p] * dot(W[row_p, 0:K], H[col_p, 0:K])     for every nonzero p of S
 *
 * S is a (row, col)-sorted sparse matrix with int32 indices and fp32 values,
 * W is n_rows x K and H is n_cols x K, both fp32 row-major; out has one fp32
 * per nonzero, in the order of the sorted S.
 *
 * The reference program (isratnisa/SDDMM_GPU) has no library interface: it is
 * one translation unit whose main() calls free functions.  Each entry point
 * below replaces one of those call sites; the citation names the reference
 * lines (relative to HiPC18/src/).  All functions return SDDMM_OK (0) or an
 * error code and never throw; sddmm_last_error() gives the message of the
 * last failure on the calling thread.  "host" / "device" say where a pointer
 * must live.  Plans are immutable after creation: sddmm_execute may be called
 * from several threads on the same plan (each call on its own stream) -- with
 * one exception: a plan that works in K slices (sddmm_plan_info.k_slice < K,
 * i.e. K > 128) keeps the partial results between its slices in a buffer of
 * its own, so executes of such a plan must not overlap in time -- unless they
 * are made through sddmm_execute_ws, which takes that memory from the caller.
 */
#ifndef SDDMM_H
#define SDDMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    SDDMM_OK = 0,
    SDDMM_ERR_ARG = 1,      /* null pointer, non-positive size, K < 1, ... */
    SDDMM_ERR_IO = 2,       /* file cannot be opened / read / written */
    SDDMM_ERR_FORMAT = 3,   /* not a coordinate Matrix Market file, short file, bad token */
    SDDMM_ERR_RANGE = 4,    /* an index outside the matrix, or sizes beyond int32 offsets */
    SDDMM_ERR_UNSORTED = 5, /* operation needs a (row, col)-sorted matrix */
    SDDMM_ERR_HIP = 6,      /* a HIP runtime call failed, or no gfx950 device */
    SDDMM_ERR_NOMEM = 7
};

/* Kernel families a plan can be pinned to (sddmm_plan_create flags, low byte).
 * AUTO lets the planner choose from the matrix shape, K and the tile sizes
 * (it builds a HYBRID plan, which may consist of a single family). */
enum {
    SDDMM_KERNEL_AUTO = 0,
    SDDMM_KERNEL_ROW_GATHER = 1, /* W row in VGPRs, H rows gathered from L2/HBM (as a plan: the unpadded stream kernel;
                                    as the short-row launch of a HYBRID plan: the padded, pipelined gather, over
                                    column slabs when H is far larger than the caches) */
    SDDMM_KERNEL_LDS_TILE = 2,   /* column tiles of H staged in LDS, W row (re)loaded per row run */
    SDDMM_KERNEL_PANEL = 3,      /* row panels of W resident in VGPRs, column tiles of H swept through LDS */
    SDDMM_KERNEL_HYBRID = 4,     /* what AUTO builds: (from K = 512 on, or when asked) the dense core as a DENSE_BLOCK
                                    launch, the rest split by row length: rows with at least 2 nonzeros per column
                                    tile -> LDS_TILE (padded tile kernel), shorter rows -> ROW_GATHER; a class too
                                    small to pay for its launch joins the other.  Never a PANEL launch. */
    SDDMM_KERNEL_DENSE_BLOCK = 5 /* blocks of 128 heavy rows x 128 popular columns computed whole on the matrix cores,
                                    their nonzeros picked from the result; never a plan of its own, only a launch of a
                                    HYBRID plan (reported by sddmm_execute_profiled) */
};

typedef struct sddmm_coo sddmm_coo;   /* host-side sparse matrix (COO, int32/int32/fp32) */
typedef struct sddmm_plan sddmm_plan; /* device-side execution plan for one (S pattern, K, tiles) */

typedef struct sddmm_plan_info {
    int64_t n_rows, n_cols, nnz;
    int64_t rows_touched, cols_touched; /* rows / columns with at least one nonzero */
    int32_t K;
    int32_t tile_size_x;  /* columns of S (= rows of H) per LDS tile actually used */
    int32_t tile_size_y;  /* row-panel height actually used */
    int32_t k_slice;      /* K elements of each H row resident in LDS at a time (== K: no slicing) */
    int32_t n_col_tiles, n_row_panels; /* (n_row_panels: row panels of the stream; with tile_runs = 2 the
                                          row ranges, one per group of workgroups) */
    int32_t kernel;       /* SDDMM_KERNEL_* actually chosen (HYBRID: more than one launch) */
    int32_t n_launches;   /* kernel launches per sddmm_execute */
    int32_t lanes_per_nnz;
    int32_t lds_bytes;    /* LDS per workgroup of the main kernel */
    int32_t grid, block;  /* launch shape of the main kernel */
    int64_t n_blocks;     /* (row panel, column tile) work items with at least one nonzero */
    int64_t device_bytes; /* device memory owned by the plan */
    int64_t class_nnz[3]; /* nonzeros handled by LDS_TILE, PANEL (explicit PANEL plans only), ROW_GATHER launches;
                             with dense_nnz they add up to nnz */
    int64_t class_rows[3];
    int64_t padded_positions; /* stream positions of the LDS_TILE launches, padding included */
    int64_t short_batches;    /* batches of 64 of those positions that run in half the steps */
    double plan_ms;       /* host time spent in the tiling pass + upload (a loaded plan: in reading the file) */
    int64_t dense_nnz;    /* nonzeros handled by the DENSE_BLOCK launch */
    int64_t dense_blocks; /* its 128 x 128 blocks */
    int64_t matrix_nnz;   /* nonzeros of the LDS_TILE launch computed by its matrix-core waves (counted in class_nnz[0]) */
    int64_t matrix_rows;  /* the rows they belong to */
    int64_t spmm_runs;    /* (row, tile) runs of the product's tile stream, one partial row of Y each (0: not built) */
} sddmm_plan_info;

const char *sddmm_last_error(void);
const char *sddmm_version(void);

/* ---------------------------------------------------------------- input --- */

/* Reads a Matrix Market coordinate file (real | integer | pattern, general |
 * symmetric; '%' comment lines; the banner line may be missing).  Indices
 * become 0-based.  Order and duplicates are kept as in the file.
 * Replaces the inline reader in main(), sddmm.cu:257-283.                   */
int sddmm_read_mtx(const char *path, sddmm_coo **out);

/* Writes S as "%%MatrixMarket matrix coordinate real general" (1-based). */
int sddmm_write_mtx(const sddmm_coo *S, const char *path);

/* Binary side-file of a parsed matrix (header + raw arrays), so large inputs
 * are parsed from text once.  The reference's analogue is the ad-hoc text
 * dump at util.h:83-118.                                                    */
int sddmm_write_bin(const sddmm_coo *S, const char *path);
int sddmm_read_bin(const char *path, sddmm_coo **out);

/* A synthetic matrix of one of the five benchmark shapes, (row, col)-sorted:
 * config 1 uniform 4096^2 at 1 %; 2 bag of words 1500 x 12,419 (lognormal row
 * lengths, Zipf(1.1) columns, counts as values); 3 recommender 480,189 x 17,770
 * (power-law row lengths, Zipf(0.9) columns, ratings 1..5; about 100 M nonzeros);
 * 4 R-MAT 2^22 (200 M edges before duplicates are removed); 5 banded 2^20 (64 per
 * row inside +-2048 of the diagonal).  scale in (0, 1] shrinks the dimensions
 * (the nonzeros shrink with them); the result depends on (config, scale, seed)
 * only, not on the number of host threads.  No counterpart in the reference,
 * whose inputs are downloaded files (HiPC18/run.sh:3-6): this is what the
 * command-line tool's --gen reads instead of a file.                          */
int sddmm_coo_generate(int32_t config, double scale, uint64_t seed, sddmm_coo **out);

/* Copies caller arrays (host) into a new matrix.  vals may be NULL (all 1). */
int sddmm_coo_create(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *rows,
                     const int32_t *cols, const float *vals, sddmm_coo **out);
void sddmm_coo_destroy(sddmm_coo *S);

int sddmm_coo_info(const sddmm_coo *S, int64_t *n_rows, int64_t *n_cols, int64_t *nnz,
                   int *is_row_col_sorted);
/* Borrowed host pointers, valid until S is modified or destroyed. */
int sddmm_coo_arrays(const sddmm_coo *S, const int32_t **rows, const int32_t **cols,
                     const float **vals);

/* Stable sort into (row, col) order; duplicates kept in file order. */
int sddmm_coo_sort_rows(sddmm_coo *S);

/* "Conversion from col sorted to row sorted": swaps the roles of rows and
 * columns (n_rows <-> n_cols) and sorts, so a column-sorted file of A comes
 * out as row-sorted A^T.  Replaces unsorted_make_CSR, util.h:82-128.        */
int sddmm_coo_transpose_sort(sddmm_coo *S);

/* CSR row pointers (n_rows+1 entries, host) of a sorted matrix. */
int sddmm_coo_row_ptr(const sddmm_coo *S, int32_t *row_ptr);

/* Compressed CSR over the non-empty rows: row_holder[h] = h-th non-empty row,
 * row_ptr[h]..row_ptr[h+1] its nonzeros.  row_ptr has room for n_rows+1,
 * row_holder for n_rows entries.  Replaces make_CSR, util.h:131-153.        */
int sddmm_coo_compress_rows(const sddmm_coo *S, int32_t *row_ptr, int32_t *row_holder,
                            int64_t *n_nonempty);

/* X[r*k+t] = 0.1*drand48() after srand48(0): the dense factors the reference
 * CLI runs with.  Replaces initial(), util.h:75-81.  X is a host pointer.   */
int sddmm_init_reference(float *X, int64_t n, int32_t k);

/* The SDDMM on the host cores: out[p] = S.val[p] * (sum over t ascending of
 * W[row_p*K+t] * H[col_p*K+t]), every sum sequential in fp32 -- the arithmetic
 * and the result, bit for bit, of sddmm_CPU_CSR / sddmm_CPU_COO
 * (sddmm.cu:153-200); nonzeros are dealt to n_threads threads (<= 0: all
 * cores), the counterpart of the reference's "#pragma omp parallel for" over
 * rows.  S must be sorted; W, H, out are host pointers (out: nnz fp32).  Needs
 * no GPU: this is what the command-line tool checks the device result
 * against, as the reference does at sddmm.cu:126-145.                       */
int sddmm_cpu(const sddmm_coo *S, int32_t K, const float *W, const float *H, float *out,
              int32_t n_threads);

/* --------------------------------------------------------------- tiling --- */

/* Host-side result of the tiling pass, for inspection and tests.  S is cut
 * into column tiles of tile_size_x columns; "tile order" lists the nonzeros
 * tile by tile, rows ascending inside a tile, columns ascending inside a row
 * -- the order rewrite_matrix_1D writes (util.h:267-343).  Nonzeros are not
 * copied: tiled_ind gives, for each tile-order position, the position in the
 * sorted S (the reference's tiled_ind, util.h:301).  Because S is (row, col)-
 * sorted, each (tile, row) run is a contiguous range of original positions.
 * Inside a tile every tile_size_y active rows (rows with a nonzero in the
 * tile) form a row panel; block_end holds the tile-order end offset of each
 * panel (the reference's lastIdx_block_tile, stored without its n_rows/Y+1
 * stride).  Replaces TiledMatrix + rewrite_matrix_1D, util.h:33-66, 267-343. */
typedef struct sddmm_tiling sddmm_tiling;
typedef struct sddmm_tiling_view {
    int32_t tile_size_x, tile_size_y, n_col_tiles;
    int32_t max_active_rows;   /* largest n_actv_row: rewrite_matrix_1D's return value */
    int64_t nnz;
    const int32_t *tile_ptr;   /* [n_col_tiles+1] tile-order offsets (lastIdx_tile) */
    const int32_t *tiled_ind;  /* [nnz] */
    const int64_t *active_ptr; /* [n_col_tiles+1]; n_actv_row[j] = active_ptr[j+1]-active_ptr[j] */
    const int32_t *active_row; /* global row ids, tile j at [active_ptr[j], active_ptr[j+1]) */
    const int32_t *active_end; /* tile-order end offset of that row's run */
    const int64_t *block_ptr;  /* [n_col_tiles+1] offsets into block_end */
    const int32_t *block_end;  /* tile-order end offset of each row panel */
} sddmm_tiling_view;
int sddmm_tiling_create(const sddmm_coo *S, int32_t tile_size_x, int32_t tile_size_y,
                        sddmm_tiling **out);
int sddmm_tiling_get(const sddmm_tiling *T, sddmm_tiling_view *view);
void sddmm_tiling_destroy(sddmm_tiling *T);

/* ----------------------------------------------------------------- plan --- */

/* Builds a plan from a sorted host matrix: runs the tiling pass for
 * (K, tile_size_x, tile_size_y), uploads index arrays and S.val.  tile sizes
 * of 0 mean "choose".  tile_size_x = columns of S per LDS tile, tile_size_y =
 * row-panel height: the 3rd and 4th positional arguments of the reference CLI
 * (README.md:21-33).  flags: low byte = SDDMM_KERNEL_*.
 * Replaces the TiledMatrix/rewrite_matrix_1D call in preprocessing()
 * (sddmm.cu:208-232) and the allocation + host-to-device part of sddmm_GPU
 * (sddmm.cu:38-73).                                                         */
int sddmm_plan_create(const sddmm_coo *S, int32_t K, int32_t tile_size_x, int32_t tile_size_y,
                      uint32_t flags, sddmm_plan **out);

/* Same, for a CSR pattern that already lives in device memory (d_row_ptr:
 * n_rows+1 int32, d_col_ind: nnz int32, sorted inside each row).  The plan
 * borrows both arrays: they must outlive it.  The tiling pass runs from a
 * host copy of the pattern made here.                                       */
int sddmm_plan_create_device(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                             const int32_t *d_col_ind, int32_t K, int32_t tile_size_x,
                             int32_t tile_size_y, uint32_t flags, sddmm_plan **out);

/* Everything that shapes a plan, for callers that want more than the two tile
 * sizes.  sddmm_plan_options_init() sets every field to "let the planner
 * choose" (-1; kernel AUTO; tile sizes 0); a plan built from the same matrix, K
 * and options is always the same plan.  Every field can also be overridden
 * from the environment (variable named in brackets, read when a plan is
 * created, unless ignore_env is set) -- a tuning aid for runs where the caller's
 * code cannot be changed; sddmm_plan_get_options() reports the values a plan
 * was actually built with, overrides included.
 *
 * tile_size_x is honoured by every LDS-tile launch (capped by what fits the
 * 160 KB LDS).  tile_size_y is the row-panel height of the PANEL kernel and of
 * an explicitly requested LDS_TILE plan, and, in the plans AUTO/HYBRID build,
 * the height of the row ranges a wide matrix is walked in (tile_runs = 2: the
 * rows are cut into at least rows / tile_size_y ranges of equal nonzero count).
 * Their other tile launches cut the rows into one block of equal nonzero count
 * per die (or per workgroup share of a tile) whatever tile_size_y says.
 * plan_info.tile_size_y reports the most rows any one block or range holds.   */
typedef struct sddmm_plan_options {
    int32_t kernel;             /* SDDMM_KERNEL_*                                   [SDDMM_KERNEL]        */
    int32_t tile_size_x;        /* columns of S per LDS tile, 0 = choose            [SDDMM_TILE_X]        */
    int32_t tile_size_y;        /* row-panel height, 0 = choose                     [SDDMM_TILE_Y]        */
    int32_t k_slice;            /* K elements per tile-kernel launch (32/64/128)    [SDDMM_TILE_KSLICE]   */
    int32_t tile_lanes;         /* lanes per nonzero of the tile kernel (4/8/16)    [SDDMM_TILE_G]        */
    int32_t tile_waves;         /* waves per workgroup of the tile kernel (12/16)   [SDDMM_TILE_WAVES]    */
    int32_t tile_assign;        /* 0 equal position ranges, 1 tile x row block,
                                   2 the same with a row block's tiles on one die   [SDDMM_TILE_ASSIGN]   */
    int32_t tile_few_blocks;    /* 0/1 fewest row blocks when staging dominates     [SDDMM_TILE_FEW_BLOCKS] */
    int32_t tile_short_batches; /* 0/1 run ends of <= lanes/2 nonzeros batched apart [SDDMM_TILE_SHORT]    */
    int32_t tile_deal;          /* 0/1 heavy and light tiles dealt to one workgroup [SDDMM_TILE_DEAL]     */
    int32_t tile_runs;          /* more tiles than workgroups: 0 tiles dealt round-robin,
                                   1 runs of neighbouring tiles to one die, 2 row ranges
                                   walked by groups of workgroups of one die (-1:
                                   2 where rows touch few tiles each, else 1)       [SDDMM_TILE_RUNS]     */
    int32_t gather_lanes;       /* lanes per nonzero of the short-row launch        [SDDMM_GATHER_G]      */
    int32_t gather_padded;      /* 0/1 short rows through the padded gather kernel  [SDDMM_GATHER_PADDED] */
    int32_t gather_sink;        /* 0/1 padding of that stream flagged and dropped   [SDDMM_GATHER_SINK]   */
    int32_t row_padded;         /* 0/1 ROW_GATHER plans use the padded gather kernel [SDDMM_ROW_PADDED]    */
    int32_t unpadded_tile;      /* 0/1 LDS_TILE plans use the unpadded stream kernel [SDDMM_UNPADDED_TILE] */
    int32_t dense_blocks;       /* 0/1 dense core on the matrix cores (-1: by K)    [SDDMM_DENSE]         */
    int32_t dense_permille;     /* least fill of a dense block, in 1/1000           [SDDMM_DENSE_PERMILLE] */
    int32_t dense_rb_group;     /* row blocks swept together by one die             [SDDMM_DENSE_RB_GROUP] */
    int32_t fuse_slices;        /* 0/1 the K slices of a launch run inside one kernel
                                   launch (-1: where the stream is small)           [SDDMM_FUSE_SLICES]   */
    int32_t matrix_rows;        /* 1: the heaviest rows of an LDS_TILE launch go, as 32 x 32
                                   blocks, to matrix-core waves inside the same workgroups
                                   (0 and -1: off: fp32 MFMA and vector work of one SIMD do
                                   not overlap, so the share measured slower)         [SDDMM_MATRIX_ROWS]   */
    int32_t matrix_permille;    /* least fill of such a row, in 1/1000 of n_cols      [SDDMM_MATRIX_PERMILLE] */
    int32_t matrix_waves;       /* matrix-core waves per workgroup: 4 (next to 12
                                   vector waves) or 8 (next to 8)                     [SDDMM_MATRIX_WAVES]  */
    int32_t spmm_stream;        /* 1: the plan also lays out its LDS_TILE launch for the product
                                   Y = X H (sddmm_plan_spmm) on the same column tiles  [SDDMM_SPMM_STREAM]   */
    int32_t ignore_env;         /* 1: the environment is not consulted                                      */
    int64_t gather_slab_cols;   /* padded gather streams S in slabs of this many columns [SDDMM_GATHER_SLAB_COLS] */
    int64_t gather_panel_rows;  /* ... and, inside, in panels of this many listed rows   [SDDMM_GATHER_PANEL_ROWS] */
    int64_t dense_min_nnz;      /* fewer dense nonzeros than this: no dense launch  [SDDMM_DENSE_MIN_NNZ] */
    int64_t panel_bytes;        /* W bytes per row panel of an LDS_TILE stream      [SDDMM_PANEL_BYTES]   */
    int64_t short_row_max;      /* rows with fewer nonzeros go to the short class   [SDDMM_SHORT_ROW_MAX] */
    int64_t stage_factor;       /* long class needs this many nonzeros per staged H row [SDDMM_STAGE_FACTOR] */
    int64_t split_min_nnz;      /* smaller matrices are one launch                  [SDDMM_SPLIT_MIN_NNZ] */
} sddmm_plan_options;
void sddmm_plan_options_init(sddmm_plan_options *opt);

/* sddmm_plan_create / sddmm_plan_create_device with the full option set
 * (opt == NULL: defaults).  No counterpart in the reference, whose only knobs
 * are the two tile sizes on the command line (sddmm.cu:253-254).             */
int sddmm_plan_create_opt(const sddmm_coo *S, int32_t K, const sddmm_plan_options *opt,
                          sddmm_plan **out);
int sddmm_plan_create_device_opt(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                                 const int32_t *d_col_ind, int32_t K, const sddmm_plan_options *opt,
                                 sddmm_plan **out);
int sddmm_plan_get_options(const sddmm_plan *plan, sddmm_plan_options *opt);

/* Plan files: the tiling pass is the expensive part of setting up a large
 * matrix (half a second at 10^8 nonzeros), so a plan can be written to a file
 * next to the matrix's binary side-file and loaded back instead of being built
 * again.  The file holds the plan's device arrays and launch descriptors under
 * a key: matrix size, nnz, K, the plan options it was built with (tile sizes
 * and kernel family among them) and a hash of the sparsity pattern.  Loading
 * checks the key against the caller's matrix, K and options (opt == NULL: any
 * options) and fails with SDDMM_ERR_FORMAT on a mismatch or on a file written
 * by another build of the library.  sddmm_plan_load is the counterpart of
 * sddmm_plan_create (the file carries the pattern and the values);
 * sddmm_plan_load_device the one of sddmm_plan_create_device (the plan borrows
 * the caller's device arrays again; the pattern hash is computed on the device).
 * The reference's analogue are the ad-hoc dumps of its converted matrices,
 * util.h:83-118.                                                             */
int sddmm_plan_save(const sddmm_plan *plan, const char *path);
int sddmm_plan_load(const char *path, const sddmm_coo *S, int32_t K, const sddmm_plan_options *opt,
                    sddmm_plan **out);
int sddmm_plan_load_device(const char *path, int64_t n_rows, int64_t n_cols, int64_t nnz,
                           const int32_t *d_row_ptr, const int32_t *d_col_ind, int32_t K,
                           const sddmm_plan_options *opt, sddmm_plan **out);

/* Gives the plan its own copy of S.val (nnz fp32 in sorted order, device
 * pointer), laid out the way each of its kernels streams the nonzeros, so
 * that sddmm_execute(plan, NULL, ...) reads values coalesced.  This is what
 * sddmm_plan_create does for a host matrix; use it after
 * sddmm_plan_create_device, or to change the values of a fixed pattern.  Runs
 * on `stream`; not to be called while an execute of the same plan is in
 * flight.  The reference uploads the values together with the tiled indices
 * (tS.vals, util.h:304, sddmm.cu:51).                                        */
int sddmm_plan_set_values(sddmm_plan *plan, const float *d_val, void *stream);

int sddmm_plan_get_info(const sddmm_plan *plan, sddmm_plan_info *info);
void sddmm_plan_destroy(sddmm_plan *plan);

/* -------------------------------------------------------------- execute --- */

/* Launches the SDDMM on `stream` (a hipStream_t, NULL = default stream) and
 * returns without synchronising.  All four pointers are device pointers:
 *   d_val  nnz fp32 in sorted order; NULL = the values uploaded with the plan
 *          (for a plan made by sddmm_plan_create_device: NULL = no scaling,
 *          out[p] = dot, the form the shipping reference kernel computes,
 *          kernel.h:47-48)
 *   d_W    n_rows*K, d_H  n_cols*K, row-major;  d_out  nnz fp32 (overwritten).
 * Replaces the launch loop of sddmm_GPU, sddmm.cu:88-108, and
 * comp_kernel_COO, kernel.h:2-52.                                           */
int sddmm_execute(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H,
                  float *d_out, void *stream);

/* sddmm_execute with the per-nonzero epilogue chosen by the caller, fused into
 * the kernels' store (no second pass over out):
 *   SDDMM_EPILOGUE_SCALE     out[p] = val[p] * dot    (= sddmm_execute; sddmm.cu:173)
 *   SDDMM_EPILOGUE_RESIDUAL  out[p] = val[p] - dot    (needs values: d_val or plan-owned)
 * The residual is the error term of the matrix-factorisation updates (ALS,
 * SGD) that the reference names as the use of SDDMM (README.md:1); the
 * reference itself computes the scaled form only.                           */
#define SDDMM_EPILOGUE_SCALE 0
#define SDDMM_EPILOGUE_RESIDUAL 1
int sddmm_execute_epilogue(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H,
                           float *d_out, int32_t epilogue, void *stream);

/* The same calls with the scratch memory brought by the caller.  A plan whose
 * launches cover K in several slices keeps partial results between the slices, a
 * launch with a matrix-core share packs its operands, and the softmax pass keeps
 * per-chunk records: sddmm_execute, sddmm_execute_epilogue and
 * sddmm_execute_softmax hold that memory in the plan (or, for the softmax
 * records, in a per-device array of the library), so two of their calls on one
 * plan must not overlap in time unless the plan needs none (one launch over all
 * of K, no softmax).  sddmm_execute_ws takes it from d_workspace instead --
 * device memory, 256-byte aligned, at least sddmm_plan_workspace_bytes(plan)
 * long, which the call may overwrite entirely and needs only until its work on
 * `stream` has finished -- and touches nothing of the plan: any number of calls
 * on one plan, each with a workspace of its own, may run at the same time (other
 * threads, other streams).  form = SDDMM_EPILOGUE_SCALE or _RESIDUAL, ored with
 * SDDMM_FORM_SOFTMAX for the row softmax of the result.  No counterpart in the
 * reference, whose sddmm_GPU allocates per call (sddmm.cu:38-73).              */
#define SDDMM_FORM_SOFTMAX 0x100
int sddmm_plan_workspace_bytes(const sddmm_plan *plan, int64_t *bytes);
int sddmm_execute_ws(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H,
                     float *d_out, int32_t form, void *d_workspace, int64_t workspace_bytes, void *stream);

/* The forms that surround an SDDMM where it is used as sparse attention or
 * in graph networks -- "SDDMM ... is a core of many machine learning
 * algorithms" (README.md:1); the reference itself stops at the sampled product.
 *
 * sddmm_execute_softmax: sddmm_execute followed, on the same stream, by the
 * row-wise softmax of the results in place:
 *   out[p] = exp(s_p - m_r) / sum_{q in row r} exp(s_q - m_r),  s = val .* (W H^T) on S's pattern,
 * m_r the row's largest s.  One extra pass over out (the row totals must be known
 * before any entry can be normalised): every row of up to 16,376 entries is
 * taken into registers whole -- by a lane, a group of lanes, a wave or a
 * workgroup, by its length -- so it is read once and written once; a longer row
 * is cut into pieces of 4096 entries whose (max, sum) records are merged by a
 * last kernel.  The layout of the work and those records are kept in fixed
 * device arrays of the library (18 MiB per GPU), so softmax calls that overlap
 * in time on one GPU (different streams or threads) race unless they bring a
 * workspace (sddmm_execute_ws); calls on one stream never do.
 * sddmm_row_softmax: the same pass on its own, over any CSR pattern in device
 * memory (d_out may be d_x; n_rows < 2^31 - 1, row_ptr[n_rows] entries).
 * sddmm_spmm_csr: Y[r, 0:K] = sum over row r's entries p of x[p] * H[col_p, 0:K]
 * (d_Y: n_rows*K fp32, overwritten; rows without entries become 0), the product
 * that consumes the attention weights.  Rows that straddle the 256-entry chunks
 * the waves work in are completed with fp32 atomic adds, so their last bits can
 * differ from run to run.
 *
 * sddmm_plan_spmm: the same product behind the plan of its SDDMM.  A plan made
 * with spmm_stream = 1 walks the rows of its LDS_TILE launch once more, as
 * (row, tile) runs: a group of 8 lanes adds x[p] * (its slice of the H row, read
 * from the column tile in LDS) over a run and writes one partial row; a second
 * kernel adds the partial rows of every row; the plan's other rows gather their
 * H rows as sddmm_spmm_csr does.  No atomics: the same bits on every call.  The
 * partial rows (K floats per run; sddmm_plan_info.spmm_runs) live in the plan, or
 * in d_workspace (NULL, or as for sddmm_execute_ws).  Other plans (and H or Y not
 * 16-byte aligned) take the sddmm_spmm_csr path on the plan's pattern.  d_x: nnz
 * fp32 in sorted order, e.g. the output of sddmm_execute_softmax.            */
int sddmm_execute_softmax(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H,
                          float *d_out, void *stream);
int sddmm_plan_spmm(const sddmm_plan *plan, const float *d_x, const float *d_H, float *d_Y, void *d_workspace,
                    int64_t workspace_bytes, void *stream);
int sddmm_row_softmax(int64_t n_rows, const int32_t *d_row_ptr, const float *d_x, float *d_out, void *stream);
int sddmm_spmm_csr(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                   const int32_t *d_col_ind, const float *d_x, int32_t K, const float *d_H, float *d_Y,
                   void *stream);

/* The same execution with an event after every launch-list entry: fills one
 * profile per entry (sddmm_plan_launch_count of them) with its wall time on
 * the device, then returns (synchronises on the last event).  No counterpart
 * in the reference, which times its whole launch loop with one event pair
 * (sddmm.cu:93-112); the bench uses it to attribute time to kernel families. */
typedef struct sddmm_launch_profile {
    int32_t kernel;            /* SDDMM_KERNEL_ROW_GATHER / LDS_TILE / PANEL */
    int32_t lanes_per_nnz;
    int32_t k_slice;           /* K elements per kernel launch */
    int32_t n_kernel_launches; /* K / k_slice */
    int64_t nnz, rows;         /* nonzeros and rows this entry covers */
    int64_t stream_positions;  /* positions walked, padding included */
    float ms;
} sddmm_launch_profile;
int sddmm_plan_launch_count(const sddmm_plan *plan, int32_t *n);
int sddmm_execute_profiled(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H,
                           float *d_out, void *stream, sddmm_launch_profile *prof, int32_t max_prof);

/* Host-pointer form with the calling convention of the reference's
 * sddmm_GPU(S, tiledS, P, W, H) (sddmm.cu:32): copies W and H to the device,
 * runs the kernels between two events, copies the result back into h_out
 * (nnz fp32, sorted order) and reports the kernel-only time in milliseconds,
 * the quantity the reference prints at sddmm.cu:109-114.                    */
int sddmm_gpu(const sddmm_plan *plan, const float *h_W, const float *h_H, float *h_out,
              float *kernel_ms);

/* Plan-free SDDMM over a CSR pattern in device memory that allocates nothing:
 * no hipMalloc / hipFree and no allocating library routine in the call.  The
 * first call of a process on a device looks up the address of the library's
 * fixed array and is the first launch of its kernels, which is when the runtime
 * may load the code object and materialise that array: make one warm-up call per
 * device outside any graph capture; after it, no call allocates.  It has
 * no counterpart in the reference (whose sddmm_GPU allocates and frees on every
 * call, sddmm.cu:38-73, 147-150); it is for callers that cannot allocate --
 * code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc -- and therefore cannot create a plan.  Same result as
 * sddmm_plan_create_device(..., SDDMM_KERNEL_ROW_GATHER) + sddmm_execute, bit
 * for bit: the row-gather kernel, whose per-batch side array (the row of every
 * 64th nonzero) is built on the device, on `stream`, into a fixed 16 MiB
 * device array of the library.  All pointers are device pointers; d_val may be
 * NULL (out[p] = dot).  The pattern is not validated (that would need a copy
 * to the host): d_row_ptr must be monotone with d_row_ptr[0] = 0 and
 * d_row_ptr[n_rows] = nnz, columns inside [0, n_cols).  nnz above SDDMM_NOALLOC_MAX_NNZ is rejected with
 * SDDMM_ERR_RANGE.  Every call on a GPU uses that GPU's one array: calls that
 * overlap in time on the same GPU (different streams or threads) race.       */
#define SDDMM_NOALLOC_MAX_NNZ (1 << 28)
int sddmm_csr_noalloc(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                      const int32_t *d_col_ind, const float *d_val, int32_t K, const float *d_W,
                      const float *d_H, float *d_out, void *stream);

/* Measurement aid: copies n_bytes (a multiple of 16, both pointers 16-byte
 * aligned device memory) with a plain streaming kernel, sddmm_copy_probe_kernel,
 * on `stream`.  A profile of a run that also calls this holds a kernel of known
 * size (n_bytes read, n_bytes written) to scale the HBM byte counters by.  No
 * counterpart in the reference.                                              */
int sddmm_copy_probe(const void *d_src, void *d_dst, int64_t n_bytes, void *stream);

/* Number of visible devices and the gcnArchName of device 0 ("" if none). */
int sddmm_device_info(int *n_devices, char *arch, int arch_len);

#ifdef __cplusplus
}
#endif
#endif /* SDDMM_H */
