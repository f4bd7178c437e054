// Device side of the SDDMM engine for gfx950 (MI355X): plan construction
// (stream descriptors for the kernels, upload) and the HIP kernels.
//
// Both kernel families walk a "stream" of nonzeros in batches of 64 (one per
// lane of a wavefront):
//   row-gather : the stream is the sorted S itself, cut into fixed chunks;
//   LDS-tile   : the stream is S in tile order (column tile by column tile,
//                rows ascending inside a tile) reached through the permutation
//                the tiling pass produced; the workgroup stages the tile's H
//                rows in LDS first.
// A batch loads its 64 column indices / values / outputs coalesced.  The rows
// of the 64 nonzeros come from two small side arrays (first segment of the
// batch + a 64-bit mask of "a new row starts here"), so no per-nonzero row
// index is read.  Inside a batch, groups of G lanes each take G consecutive
// nonzeros: for each, the group reads the H row (from LDS or global) as
// contiguous 16-byte pieces, multiplies with the W row slice it keeps in
// VGPRs while the row lasts, and the G partial sums of G nonzeros are reduced
// together by a butterfly of cross-lane exchanges that leaves nonzero i's dot
// product in lane i, which scales it by S.val and stores it.
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstring>
#include <new>
#include "internal.hpp"

using namespace sddmm;

namespace {

struct WorkItem {
    int32_t begin, end;   // stream positions
    int32_t batch_base;   // index of the item's first batch in batch_seg / batch_mask
    int32_t tile;         // column tile staged in LDS (-1: none)
};

struct KArgs {
    const int32_t *col_ind;    // [nnz] sorted order
    const float *val;          // [nnz] or null (no scaling)
    const float *W, *H;
    float *out;
    const int32_t *perm;       // stream position -> sorted position, null = identity
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
};

constexpr int kRowGatherBlock = 256;   // 4 waves
constexpr int kRowGatherBatchesPerWave = 8;
constexpr int kLdsBlock = 1024;        // 16 waves, one workgroup per CU
constexpr int kLdsMaxBytes = 160 * 1024;

__device__ __forceinline__ float dot4(const float4 &a, const float4 &b, float acc)
{
    acc = fmaf(a.x, b.x, acc);
    acc = fmaf(a.y, b.y, acc);
    acc = fmaf(a.z, b.z, acc);
    acc = fmaf(a.w, b.w, acc);
    return acc;
}

// Reduces G accumulators across the G lanes of a group so that lane i of the
// group ends with the full sum of accumulator i (returned).
template <int G>
__device__ __forceinline__ float transpose_reduce(float (&acc)[G], int l)
{
#pragma unroll
    for (int s = G / 2; s >= 1; s >>= 1) {
        const bool upper = (l & s) != 0;
#pragma unroll
        for (int j = 0; j < s; ++j) {
            float keep = upper ? acc[j + s] : acc[j];
            float send = upper ? acc[j] : acc[j + s];
            acc[j] = keep + __shfl_xor(send, s, G);
        }
    }
    return acc[0];
}

// K = 4 * (number of float4 per row); each lane of a group owns KPL float4
// slots of a row: slot j sits at float4 index (((j + rot) % KPL) * G + l).  `rot`
// differs between the groups that share one 16-lane LDS access phase, so that
// their 16-byte reads fall into different banks when rows are a multiple of
// 256 bytes apart.  EXACT: K == 4*G*KPL (no slot is out of range).
template <int G, int KPL, bool EXACT, bool LDS_TILE>
__global__ __launch_bounds__(LDS_TILE ? kLdsBlock : kRowGatherBlock)
void sddmm_stream_kernel(const KArgs a)
{
    extern __shared__ float4 lds_tile[];
    constexpr int NW = (LDS_TILE ? kLdsBlock : kRowGatherBlock) / 64;
    constexpr int PHASE_GROUPS = (16 / G) >= 1 ? (16 / G) : 1;
    constexpr int ROT_MASK = (PHASE_GROUPS < KPL ? PHASE_GROUPS : KPL) - 1;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l = lane & (G - 1);
    const int rot = (lane / G) & ROT_MASK;
    const int K4 = a.K >> 2;

    int slot[KPL];
#pragma unroll
    for (int j = 0; j < KPL; ++j) slot[j] = (((j + rot) % KPL) * G + l);

    const float4 *__restrict__ W4 = reinterpret_cast<const float4 *>(a.W);
    const float4 *__restrict__ H4 = reinterpret_cast<const float4 *>(a.H);

    int item0, item1;
    if (LDS_TILE) {  // contiguous run of items per workgroup: the tile changes rarely
        item0 = (int)((int64_t)a.n_items * blockIdx.x / gridDim.x);
        item1 = (int)((int64_t)a.n_items * (blockIdx.x + 1) / gridDim.x);
    } else {
        item0 = blockIdx.x;
        item1 = item0 + 1;
    }
    int cur_tile = -1;
    int tile_base = 0;

    for (int it = item0; it < item1; ++it) {
        int begin, end, batch_base;
        if (LDS_TILE) {
            const WorkItem wi = a.items[it];
            begin = wi.begin; end = wi.end; batch_base = wi.batch_base;
            if (wi.tile != cur_tile) {
                __syncthreads();  // everyone is done with the previous tile
                cur_tile = wi.tile;
                tile_base = cur_tile * a.tile_x;
                int rows = min(a.tile_x, a.n_cols - tile_base);
                const float4 *src = H4 + (size_t)tile_base * K4;
                const int n4 = rows * K4;
                for (int i = threadIdx.x; i < n4; i += blockDim.x) lds_tile[i] = src[i];
                __syncthreads();
            }
        } else {
            begin = it * a.chunk;
            end = min(a.nnz, begin + a.chunk);
            batch_base = begin >> 6;
        }
        const int nb = (end - begin + 63) >> 6;
        const int b0 = (int)((int64_t)nb * wave / NW), b1 = (int)((int64_t)nb * (wave + 1) / NW);

        int cur_row = -1;
        float4 w[KPL];
#pragma unroll
        for (int j = 0; j < KPL; ++j) w[j] = make_float4(0.f, 0.f, 0.f, 0.f);

        for (int bi = b0; bi < b1; ++bi) {
            const int pos = begin + (bi << 6) + lane;
            const bool valid = pos < end;
            const int gb = batch_base + bi;
            const int seg0 = a.batch_seg[gb];
            const uint64_t mask = a.batch_mask[gb];
            const uint64_t le = (lane == 63) ? ~0ull : ((2ull << lane) - 1ull);
            const int seg = seg0 + __popcll(mask & le);
            int row = -1, p = 0, col = 0;
            float v = 0.f;
            if (valid) {
                row = a.seg_row ? a.seg_row[seg] : seg;
                p = a.perm ? a.perm[pos] : pos;
                col = a.col_ind[p];
                v = a.val ? a.val[p] : 1.0f;
            }
            float acc[G];
#pragma unroll
            for (int i = 0; i < G; ++i) acc[i] = 0.f;

            const int row_first = __shfl(row, 0, G);
            const int row_last = __shfl(row, G - 1, G);
            if (row_first == row_last && row_last >= 0) {
                // all G nonzeros of this group lie in one row: no checks inside
                if (row_first != cur_row) {
                    cur_row = row_first;
                    const float4 *wr = W4 + (size_t)cur_row * K4;
#pragma unroll
                    for (int j = 0; j < KPL; ++j)
                        w[j] = (EXACT || slot[j] < K4) ? wr[slot[j]] : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int i = 0; i < G; ++i) {
                    const int c_i = __shfl(col, i, G);
                    const float4 *hr = LDS_TILE ? (lds_tile + (size_t)(c_i - tile_base) * K4)
                                                : (H4 + (size_t)c_i * K4);
#pragma unroll
                    for (int j = 0; j < KPL; ++j)
                        if (EXACT || slot[j] < K4) acc[i] = dot4(w[j], hr[slot[j]], acc[i]);
                }
            } else {
#pragma unroll
                for (int i = 0; i < G; ++i) {
                    const int r_i = __shfl(row, i, G);
                    const int c_i = __shfl(col, i, G);
                    if (r_i >= 0) {
                        if (r_i != cur_row) {
                            cur_row = r_i;
                            const float4 *wr = W4 + (size_t)cur_row * K4;
#pragma unroll
                            for (int j = 0; j < KPL; ++j)
                                w[j] = (EXACT || slot[j] < K4) ? wr[slot[j]] : make_float4(0.f, 0.f, 0.f, 0.f);
                        }
                        const float4 *hr = LDS_TILE ? (lds_tile + (size_t)(c_i - tile_base) * K4)
                                                    : (H4 + (size_t)c_i * K4);
#pragma unroll
                        for (int j = 0; j < KPL; ++j)
                            if (EXACT || slot[j] < K4) acc[i] = dot4(w[j], hr[slot[j]], acc[i]);
                    }
                }
            }
            const float sum = transpose_reduce<G>(acc, l);
            if (valid) a.out[p] = sum * v;
        }
    }
}

// Any K >= 1: 8 lanes per nonzero striding over the row one float at a time,
// W re-read through the cache.  The slow, always-correct path.
__global__ __launch_bounds__(kRowGatherBlock)
void sddmm_generic_kernel(const KArgs a)
{
    constexpr int G = 8;
    constexpr int NW = kRowGatherBlock / 64;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l = lane & (G - 1);
    const int begin = blockIdx.x * a.chunk;
    const int end = min(a.nnz, begin + a.chunk);
    const int batch_base = begin >> 6;
    const int nb = (end - begin + 63) >> 6;
    const int b0 = (int)((int64_t)nb * wave / NW), b1 = (int)((int64_t)nb * (wave + 1) / NW);
    for (int bi = b0; bi < b1; ++bi) {
        const int pos = begin + (bi << 6) + lane;
        const bool valid = pos < end;
        const int gb = batch_base + bi;
        const uint64_t mask = a.batch_mask[gb];
        const uint64_t le = (lane == 63) ? ~0ull : ((2ull << lane) - 1ull);
        const int seg = a.batch_seg[gb] + __popcll(mask & le);
        int row = -1, col = 0;
        float v = 0.f;
        if (valid) {
            row = a.seg_row ? a.seg_row[seg] : seg;
            col = a.col_ind[pos];
            v = a.val ? a.val[pos] : 1.0f;
        }
        float acc[G];
#pragma unroll
        for (int i = 0; i < G; ++i) {
            const int r_i = __shfl(row, i, G);
            const int c_i = __shfl(col, i, G);
            float s = 0.f;
            if (r_i >= 0) {
                const float *wr = a.W + (size_t)r_i * a.K;
                const float *hr = a.H + (size_t)c_i * a.K;
                for (int t = l; t < a.K; t += G) s = fmaf(wr[t], hr[t], s);
            }
            acc[i] = s;
        }
        const float sum = transpose_reduce<G>(acc, l);
        if (valid) a.out[pos] = sum * v;
    }
}

struct Variant {
    int G, KPL;
    bool exact;
};

// lanes per nonzero and float4 slots per lane for a given K (K % 4 == 0)
Variant pick_variant(int K)
{
    const int K4 = K / 4;
    const int cand[][2] = {{8, 1}, {8, 2}, {8, 3}, {8, 4}, {8, 6}, {8, 8}, {16, 6}, {16, 8}, {32, 6}, {32, 8}, {64, 6}, {64, 8}};
    for (auto &c : cand)
        if (c[0] * c[1] == K4) return {c[0], c[1], true};
    for (auto &c : cand)
        if (c[0] * c[1] >= K4) return {c[0], c[1], false};
    return {0, 0, false};  // K > 2048: generic kernel
}

using KernelFn = void (*)(const KArgs);

template <bool LDS_TILE>
KernelFn lookup(const Variant &v)
{
#define SDDMM_CASE(g, kpl)                                                              \
    if (v.G == g && v.KPL == kpl)                                                       \
        return v.exact ? (KernelFn)sddmm_stream_kernel<g, kpl, true, LDS_TILE>          \
                       : (KernelFn)sddmm_stream_kernel<g, kpl, false, LDS_TILE>;
    SDDMM_CASE(8, 1) SDDMM_CASE(8, 2) SDDMM_CASE(8, 3) SDDMM_CASE(8, 4) SDDMM_CASE(8, 6) SDDMM_CASE(8, 8)
    SDDMM_CASE(16, 6) SDDMM_CASE(16, 8) SDDMM_CASE(32, 6) SDDMM_CASE(32, 8) SDDMM_CASE(64, 6) SDDMM_CASE(64, 8)
#undef SDDMM_CASE
    return nullptr;
}

#define HIP_TRY(expr)                                                                               \
    do {                                                                                            \
        hipError_t e_ = (expr);                                                                     \
        if (e_ != hipSuccess)                                                                       \
            return fail(SDDMM_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
    } while (0)

template <class T>
int upload(T **dst, const std::vector<T> &src, int64_t *bytes)
{
    *dst = nullptr;
    if (src.empty()) return SDDMM_OK;
    HIP_TRY(hipMalloc((void **)dst, src.size() * sizeof(T)));
    HIP_TRY(hipMemcpy(*dst, src.data(), src.size() * sizeof(T), hipMemcpyHostToDevice));
    *bytes += (int64_t)(src.size() * sizeof(T));
    return SDDMM_OK;
}

}  // namespace

struct sddmm_plan {
    sddmm_plan_info info{};
    Variant variant{0, 0, false};
    KernelFn fn = nullptr;
    const int32_t *d_col = nullptr;
    bool own_col = false;
    float *d_val = nullptr;
    int32_t *d_perm = nullptr, *d_seg_row = nullptr, *d_batch_seg = nullptr;
    uint64_t *d_batch_mask = nullptr;
    WorkItem *d_items = nullptr;
    int32_t n_items = 0;
    int32_t chunk = 0;
    ~sddmm_plan()
    {
        if (own_col && d_col) (void)hipFree((void *)d_col);
        if (d_val) (void)hipFree(d_val);
        if (d_perm) (void)hipFree(d_perm);
        if (d_seg_row) (void)hipFree(d_seg_row);
        if (d_batch_seg) (void)hipFree(d_batch_seg);
        if (d_batch_mask) (void)hipFree(d_batch_mask);
        if (d_items) (void)hipFree(d_items);
    }
};

namespace {

// Batch side arrays for a stream whose segment s covers stream positions
// [seg_end[s-1], seg_end[s]) (seg_end increasing, last == stream length), for
// the batches of the given items.
void build_batches(const std::vector<WorkItem> &items, const int32_t *seg_end, int64_t n_seg,
                   std::vector<int32_t> &batch_seg, std::vector<uint64_t> &batch_mask)
{
    int64_t nb_total = 0;
    if (!items.empty()) {
        const WorkItem &last = items.back();
        nb_total = last.batch_base + ((int64_t)last.end - last.begin + 63) / 64;
    }
    batch_seg.assign((size_t)nb_total, 0);
    batch_mask.assign((size_t)nb_total, 0);
    parallel_ranges((int64_t)items.size(), 4, [&](int64_t ib, int64_t ie, int) {
        for (int64_t k = ib; k < ie; ++k) {
            const WorkItem &wi = items[k];
            if (wi.end <= wi.begin) continue;
            int64_t s = std::upper_bound(seg_end, seg_end + n_seg, wi.begin) - seg_end;  // segment of wi.begin
            int64_t nb = ((int64_t)wi.end - wi.begin + 63) / 64;
            for (int64_t b = 0; b < nb; ++b) {
                int64_t p0 = wi.begin + b * 64, p1 = std::min<int64_t>(p0 + 64, wi.end);
                while (s < n_seg && seg_end[s] <= p0) ++s;
                batch_seg[wi.batch_base + b] = (int32_t)s;
                uint64_t m = 0;
                int64_t t = s;
                while (t < n_seg && seg_end[t] < p1) {  // segment t+1 starts at seg_end[t], inside (p0, p1)
                    if (seg_end[t] > p0) m |= 1ull << (seg_end[t] - p0);
                    ++t;
                }
                batch_mask[wi.batch_base + b] = m;
            }
        }
    });
}

int count_touched(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr, const int32_t *col_ind,
                  int64_t *rows_touched, int64_t *cols_touched)
{
    int64_t rt = 0;
    for (int64_t r = 0; r < n_rows; ++r) rt += row_ptr[r + 1] > row_ptr[r];
    std::vector<uint8_t> seen((size_t)n_cols, 0);
    parallel_ranges(nnz, 1 << 16, [&](int64_t b, int64_t e, int) {
        for (int64_t i = b; i < e; ++i) __atomic_store_n(&seen[col_ind[i]], (uint8_t)1, __ATOMIC_RELAXED);
    });
    int64_t ct = 0;
    for (int64_t c = 0; c < n_cols; ++c) ct += seen[c];
    *rows_touched = rt;
    *cols_touched = ct;
    return SDDMM_OK;
}

int device_ok()
{
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n < 1)
        return fail(SDDMM_ERR_HIP, "no HIP device available (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    return SDDMM_OK;
}

// Common plan builder from host CSR arrays.  d_col_borrowed != null: the
// device already holds col_ind.
int make_plan(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *row_ptr, const int32_t *col_ind,
              const float *vals, const int32_t *d_col_borrowed, int32_t K, int32_t tile_x, int32_t tile_y,
              uint32_t flags, sddmm_plan **out)
{
    auto t0 = std::chrono::steady_clock::now();
    if (K < 1) return fail(SDDMM_ERR_ARG, "plan: K must be >= 1 (got %d)", K);
    if (tile_x < 0 || tile_y < 0) return fail(SDDMM_ERR_ARG, "plan: tile sizes must be >= 0");
    if (nnz >= INT32_MAX - 4096 || n_rows >= INT32_MAX || n_cols >= INT32_MAX)
        return fail(SDDMM_ERR_RANGE, "plan: sizes beyond int32 offsets");
    if ((n_rows * (int64_t)K) >= (int64_t)1 << 40 || (n_cols * (int64_t)K) >= (int64_t)1 << 40)
        return fail(SDDMM_ERR_RANGE, "plan: dense factor too large");
    if (int rc = device_ok()) return rc;
    int want = (int)(flags & 0xff);
    if (want > SDDMM_KERNEL_LDS_TILE) return fail(SDDMM_ERR_ARG, "plan: unknown kernel id %d", want);

    sddmm_plan *P = new (std::nothrow) sddmm_plan;
    if (!P) return fail(SDDMM_ERR_NOMEM, "plan: out of memory");
    struct Guard { sddmm_plan *p; ~Guard() { delete p; } } guard{P};
    sddmm_plan_info &I = P->info;
    I.n_rows = n_rows; I.n_cols = n_cols; I.nnz = nnz; I.K = K; I.k_slice = K;
    count_touched(n_rows, n_cols, nnz, row_ptr, col_ind, &I.rows_touched, &I.cols_touched);

    const bool vec4 = (K % 4 == 0);
    Variant var = vec4 ? pick_variant(K) : Variant{0, 0, false};
    const bool have_fast = var.G != 0;

    // kernel choice
    int kernel = want;
    const int64_t row_bytes = (int64_t)K * 4;
    int32_t fit_x = (int32_t)std::min<int64_t>(kLdsMaxBytes / row_bytes, INT32_MAX);
    if (kernel == SDDMM_KERNEL_AUTO)
        kernel = (have_fast && tile_x > 0 && tile_x < n_cols && fit_x >= 8) ? SDDMM_KERNEL_LDS_TILE : SDDMM_KERNEL_ROW_GATHER;
    if (kernel == SDDMM_KERNEL_LDS_TILE && (!have_fast || fit_x < 1)) kernel = SDDMM_KERNEL_ROW_GATHER;
    I.kernel = kernel;
    I.lanes_per_nnz = have_fast ? var.G : 8;
    P->variant = var;

    int64_t dev_bytes = 0;
    if (d_col_borrowed) {
        P->d_col = d_col_borrowed;
    } else {
        int32_t *d = nullptr;
        if (nnz) {
            HIP_TRY(hipMalloc((void **)&d, (size_t)nnz * 4));
            HIP_TRY(hipMemcpy(d, col_ind, (size_t)nnz * 4, hipMemcpyHostToDevice));
            dev_bytes += nnz * 4;
        }
        P->d_col = d; P->own_col = true;
    }
    if (vals && nnz) {
        HIP_TRY(hipMalloc((void **)&P->d_val, (size_t)nnz * 4));
        HIP_TRY(hipMemcpy(P->d_val, vals, (size_t)nnz * 4, hipMemcpyHostToDevice));
        dev_bytes += nnz * 4;
    }

    std::vector<int32_t> batch_seg;
    std::vector<uint64_t> batch_mask;
    if (kernel == SDDMM_KERNEL_ROW_GATHER) {
        // segments = non-empty rows
        std::vector<int32_t> seg_end, seg_row;
        seg_end.reserve((size_t)I.rows_touched); seg_row.reserve((size_t)I.rows_touched);
        for (int64_t r = 0; r < n_rows; ++r)
            if (row_ptr[r + 1] > row_ptr[r]) { seg_end.push_back(row_ptr[r + 1]); seg_row.push_back((int32_t)r); }
        P->chunk = 64 * kRowGatherBatchesPerWave * (kRowGatherBlock / 64);
        std::vector<WorkItem> one{{0, (int32_t)nnz, 0, -1}};  // batches are global multiples of 64
        build_batches(one, seg_end.data(), (int64_t)seg_end.size(), batch_seg, batch_mask);
        if (I.rows_touched != n_rows)
            if (int rc = upload(&P->d_seg_row, seg_row, &dev_bytes)) return rc;
        I.tile_size_x = (int32_t)std::min<int64_t>(n_cols, INT32_MAX); I.tile_size_y = (int32_t)std::min<int64_t>(n_rows, INT32_MAX);
        I.n_col_tiles = 1; I.n_row_panels = 1; I.n_blocks = 1;
        I.grid = (int32_t)((nnz + P->chunk - 1) / P->chunk);
        I.block = kRowGatherBlock; I.lds_bytes = 0;
        P->fn = have_fast ? lookup<false>(var) : (KernelFn)sddmm_generic_kernel;
    } else {
        int32_t x = tile_x > 0 ? tile_x : fit_x;
        x = std::min(x, fit_x);
        x = (int32_t)std::min<int64_t>(x, std::max<int64_t>(n_cols, 1));
        int32_t y = tile_y > 0 ? tile_y : (int32_t)std::min<int64_t>(std::max<int64_t>(n_rows, 1), INT32_MAX);
        sddmm_tiling T;
        if (int rc = build_tiling(n_rows, n_cols, nnz, row_ptr, col_ind, x, y, T)) return rc;
        // work items: row panels, cut further so that no item exceeds max_item nonzeros
        const int64_t max_item = std::max<int64_t>(64 * 16 * 4, 8 * (int64_t)x);
        std::vector<WorkItem> items;
        int64_t nbatch = 0, n_blocks = 0;
        for (int32_t j = 0; j < T.n_tiles; ++j) {
            int64_t begin = T.tile_ptr[j];
            for (int64_t b = T.block_ptr[j]; b < T.block_ptr[j + 1]; ++b) {
                int64_t end = T.block_end[b];
                ++n_blocks;
                int64_t parts = std::max<int64_t>(1, (end - begin + max_item - 1) / max_item);
                int64_t per = (((end - begin + parts - 1) / parts) + 63) / 64 * 64;
                for (int64_t s = begin; s < end; s += per) {
                    int64_t e = std::min(end, s + per);
                    items.push_back({(int32_t)s, (int32_t)e, (int32_t)nbatch, j});
                    nbatch += (e - s + 63) / 64;
                }
                begin = end;
            }
        }
        build_batches(items, T.active_end.data(), (int64_t)T.active_end.size(), batch_seg, batch_mask);
        if (int rc = upload(&P->d_perm, T.tiled_ind, &dev_bytes)) return rc;
        if (int rc = upload(&P->d_seg_row, T.active_row, &dev_bytes)) return rc;
        if (int rc = upload(&P->d_items, items, &dev_bytes)) return rc;
        P->n_items = (int32_t)items.size();
        I.tile_size_x = x; I.tile_size_y = y; I.n_col_tiles = T.n_tiles;
        I.n_row_panels = (int32_t)((T.max_active_rows + y - 1) / y);
        I.n_blocks = n_blocks;
        hipDeviceProp_t prop;
        HIP_TRY(hipGetDeviceProperties(&prop, 0));
        int cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        I.grid = (int32_t)std::max<int64_t>(1, std::min<int64_t>((int64_t)cus, (int64_t)items.size()));
        I.block = kLdsBlock;
        I.lds_bytes = (int32_t)((int64_t)x * row_bytes);
        P->fn = lookup<true>(var);
        HIP_TRY(hipFuncSetAttribute((const void *)P->fn, hipFuncAttributeMaxDynamicSharedMemorySize, I.lds_bytes));
    }
    if (!P->fn) return fail(SDDMM_ERR_ARG, "plan: no kernel for K = %d", K);
    if (int rc = upload(&P->d_batch_seg, batch_seg, &dev_bytes)) return rc;
    if (int rc = upload(&P->d_batch_mask, batch_mask, &dev_bytes)) return rc;
    I.device_bytes = dev_bytes;
    I.plan_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    guard.p = nullptr;
    *out = P;
    return SDDMM_OK;
}

}  // namespace

extern "C" {

int sddmm_plan_create(const sddmm_coo *S, int32_t K, int32_t tile_size_x, int32_t tile_size_y, uint32_t flags,
                      sddmm_plan **out)
{
    if (!S || !out) return fail(SDDMM_ERR_ARG, "sddmm_plan_create: NULL argument");
    *out = nullptr;
    if (S->sorted < 0) const_cast<sddmm_coo *>(S)->sorted = check_sorted(*S) ? 1 : 0;
    if (S->sorted != 1) return fail(SDDMM_ERR_UNSORTED, "sddmm_plan_create: matrix is not (row, col)-sorted; call sddmm_coo_sort_rows");
    try {
        std::vector<int32_t> rp;
        build_row_ptr(*S, rp);
        return make_plan(S->n_rows, S->n_cols, S->nnz, rp.data(), S->cols.data(), S->vals.data(), nullptr, K,
                         tile_size_x, tile_size_y, flags, out);
    } catch (const std::bad_alloc &) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_create: out of host memory");
    }
}

int sddmm_plan_create_device(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                             const int32_t *d_col_ind, int32_t K, int32_t tile_size_x, int32_t tile_size_y,
                             uint32_t flags, sddmm_plan **out)
{
    if (!out) return fail(SDDMM_ERR_ARG, "sddmm_plan_create_device: out is NULL");
    *out = nullptr;
    if (n_rows < 0 || n_cols < 0 || nnz < 0 || !d_row_ptr || (nnz > 0 && !d_col_ind))
        return fail(SDDMM_ERR_ARG, "sddmm_plan_create_device: bad sizes or NULL arrays");
    if (nnz >= INT32_MAX - 4096 || n_rows >= INT32_MAX || n_cols >= INT32_MAX)
        return fail(SDDMM_ERR_RANGE, "sddmm_plan_create_device: sizes beyond int32 offsets");
    if (int rc = device_ok()) return rc;
    try {
        std::vector<int32_t> rp((size_t)n_rows + 1), ci((size_t)nnz);
        HIP_TRY(hipMemcpy(rp.data(), d_row_ptr, rp.size() * 4, hipMemcpyDeviceToHost));
        if (nnz) HIP_TRY(hipMemcpy(ci.data(), d_col_ind, ci.size() * 4, hipMemcpyDeviceToHost));
        if (rp[0] != 0 || rp[(size_t)n_rows] != nnz)
            return fail(SDDMM_ERR_ARG, "sddmm_plan_create_device: row_ptr does not span [0, nnz]");
        std::vector<char> bad((size_t)hw_threads() + 1, 0);
        parallel_ranges(n_rows, 1 << 12, [&](int64_t b, int64_t e, int t) {
            for (int64_t r = b; r < e; ++r) {
                if (rp[r + 1] < rp[r]) { bad[t] = 1; return; }
                for (int64_t i = rp[r]; i < rp[r + 1]; ++i) {
                    if (ci[i] < 0 || ci[i] >= n_cols) { bad[t] = 2; return; }
                    if (i > rp[r] && ci[i] < ci[i - 1]) { bad[t] = 3; return; }
                }
            }
        });
        for (char c : bad) {
            if (c == 1) return fail(SDDMM_ERR_ARG, "sddmm_plan_create_device: row_ptr is not monotone");
            if (c == 2) return fail(SDDMM_ERR_RANGE, "sddmm_plan_create_device: a column index lies outside the matrix");
            if (c == 3) return fail(SDDMM_ERR_UNSORTED, "sddmm_plan_create_device: columns are not sorted inside a row");
        }
        return make_plan(n_rows, n_cols, nnz, rp.data(), ci.data(), nullptr, d_col_ind, K, tile_size_x, tile_size_y,
                         flags, out);
    } catch (const std::bad_alloc &) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_create_device: out of host memory");
    }
}

int sddmm_plan_get_info(const sddmm_plan *plan, sddmm_plan_info *info)
{
    if (!plan || !info) return fail(SDDMM_ERR_ARG, "sddmm_plan_get_info: NULL argument");
    *info = plan->info;
    return SDDMM_OK;
}

void sddmm_plan_destroy(sddmm_plan *plan) { delete plan; }

int sddmm_execute(const sddmm_plan *plan, const float *d_val, const float *d_W, const float *d_H, float *d_out,
                  void *stream)
{
    if (!plan) return fail(SDDMM_ERR_ARG, "sddmm_execute: plan is NULL");
    const sddmm_plan_info &I = plan->info;
    if (I.nnz == 0) return SDDMM_OK;
    if (!d_W || !d_H || !d_out) return fail(SDDMM_ERR_ARG, "sddmm_execute: NULL device pointer");
    if (((uintptr_t)d_W | (uintptr_t)d_H) & 15u)
        if (I.K % 4 == 0 && plan->variant.G)
            return fail(SDDMM_ERR_ARG, "sddmm_execute: W and H must be 16-byte aligned");
    KArgs a{};
    a.col_ind = plan->d_col;
    a.val = d_val ? d_val : plan->d_val;
    a.W = d_W; a.H = d_H; a.out = d_out;
    a.perm = plan->d_perm;
    a.seg_row = plan->d_seg_row;
    a.batch_seg = plan->d_batch_seg;
    a.batch_mask = plan->d_batch_mask;
    a.items = plan->d_items;
    a.n_items = plan->n_items;
    a.nnz = (int32_t)I.nnz;
    a.chunk = plan->chunk;
    a.K = I.K;
    a.tile_x = I.tile_size_x;
    a.n_cols = (int32_t)I.n_cols;
    hipLaunchKernelGGL(plan->fn, dim3((unsigned)I.grid), dim3((unsigned)I.block), (size_t)I.lds_bytes,
                       (hipStream_t)stream, a);
    HIP_TRY(hipGetLastError());
    return SDDMM_OK;
}

int sddmm_gpu(const sddmm_plan *plan, const float *h_W, const float *h_H, float *h_out, float *kernel_ms)
{
    if (!plan || !h_W || !h_H || !h_out) return fail(SDDMM_ERR_ARG, "sddmm_gpu: NULL argument");
    const sddmm_plan_info &I = plan->info;
    float *dW = nullptr, *dH = nullptr, *dO = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    struct Free {
        float *&a, *&b, *&c; hipEvent_t &e0, &e1;
        ~Free() { if (a) (void)hipFree(a); if (b) (void)hipFree(b); if (c) (void)hipFree(c);
                  if (e0) (void)hipEventDestroy(e0); if (e1) (void)hipEventDestroy(e1); }
    } fr{dW, dH, dO, e0, e1};
    const size_t wb = (size_t)std::max<int64_t>(I.n_rows * (int64_t)I.K, 1) * 4, hb = (size_t)std::max<int64_t>(I.n_cols * (int64_t)I.K, 1) * 4;
    const size_t ob = (size_t)std::max<int64_t>(I.nnz, 1) * 4;
    HIP_TRY(hipMalloc((void **)&dW, wb));
    HIP_TRY(hipMalloc((void **)&dH, hb));
    HIP_TRY(hipMalloc((void **)&dO, ob));
    HIP_TRY(hipMemcpy(dW, h_W, (size_t)I.n_rows * I.K * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(dH, h_H, (size_t)I.n_cols * I.K * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipEventCreate(&e0));
    HIP_TRY(hipEventCreate(&e1));
    HIP_TRY(hipEventRecord(e0, nullptr));
    if (int rc = sddmm_execute(plan, nullptr, dW, dH, dO, nullptr)) return rc;
    HIP_TRY(hipEventRecord(e1, nullptr));
    HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    if (kernel_ms) *kernel_ms = ms;
    HIP_TRY(hipMemcpy(h_out, dO, (size_t)I.nnz * 4, hipMemcpyDeviceToHost));
    return SDDMM_OK;
}

int sddmm_device_info(int *n_devices, char *arch, int arch_len)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) n = 0;
    if (n_devices) *n_devices = n;
    if (arch && arch_len > 0) {
        arch[0] = 0;
        if (n > 0) {
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, 0) == hipSuccess) {
                strncpy(arch, prop.gcnArchName, (size_t)arch_len - 1);
                arch[arch_len - 1] = 0;
            }
        }
    }
    return SDDMM_OK;
}

}  // extern "C"
