// Stream kernels of the SDDMM engine for gfx950 (MI355X).
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
#include <algorithm>
#include <utility>
#include "kernels.hpp"

using namespace sddmm;

namespace {

__device__ __forceinline__ float dot4(const float4 &a, const float4 &b, float acc)
{
    acc = fmaf(a.x, b.x, acc);
    acc = fmaf(a.y, b.y, acc);
    acc = fmaf(a.z, b.z, acc);
    acc = fmaf(a.w, b.w, acc);
    return acc;
}

// value held by lane I of the caller's group of G lanes
template <int G, int I>
__device__ __forceinline__ int group_bcast(int v)
{
    if constexpr (G <= 32)
        return __builtin_amdgcn_ds_swizzle(v, (I << 5) | (0x1f & ~(G - 1)));  // src = (lane & ~(G-1)) | I
    else
        return __shfl(v, I, G);
}

// value of lane (lane ^ S)
template <int S>
__device__ __forceinline__ float xor_lane(float v)
{
    if constexpr (S == 1)
        return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
    else if constexpr (S == 2)
        return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
    else if constexpr (S < 32)
        return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (S << 10) | 0x1f));
    else
        return __shfl_xor(v, S, 64);
}

// Reduces G accumulators across the G lanes of a group so that lane i of the
// group ends with the full sum of accumulator i (returned).
template <int G, int S = G / 2>
__device__ __forceinline__ void transpose_reduce_step(float (&acc)[G], int l)
{
    if constexpr (S >= 1) {
        const bool upper = (l & S) != 0;
#pragma unroll
        for (int j = 0; j < S; ++j) {
            float keep = upper ? acc[j + S] : acc[j];
            float send = upper ? acc[j] : acc[j + S];
            acc[j] = keep + xor_lane<S>(send);
        }
        transpose_reduce_step<G, S / 2>(acc, l);
    }
}
template <int G>
__device__ __forceinline__ float transpose_reduce(float (&acc)[G], int l)
{
    transpose_reduce_step<G>(acc, l);
    return acc[0];
}

struct Batch {
    int row, p, col;  // row < 0: lane holds no nonzero
    float v;
};

// Row (segment) of stream position pos, which lies in batch gb.  With the plan's side
// arrays: the batch's first segment plus the number of segment starts up to this lane.
// Plan-free form: the largest row r between the rows of this batch's and the next
// batch's first positions with row_ptr[r] <= pos (empty rows in between never qualify
// as the largest).
__device__ __forceinline__ int segment_of(const KArgs &a, int gb, int pos, uint64_t le)
{
    if (a.batch_row) {
        int lo = a.batch_row[gb];
        int hi = (gb + 1 < ((a.nnz + 63) >> 6)) ? a.batch_row[gb + 1] : a.n_rows - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (a.row_ptr[mid] <= pos) lo = mid; else hi = mid - 1;
        }
        return lo;
    }
    return a.batch_seg[gb] + __popcll(a.batch_mask[gb] & le);
}

// K = 4 * (number of float4 per row); each lane of a group owns KPL float4
// slots of a row: slot j sits at float4 index (((j + rot) % KPL) * G + l).  `rot`
// differs between the groups that share one 16-lane LDS access phase, so that
// their 16-byte reads fall into different banks when rows are a multiple of
// 256 bytes apart.  EXACT: K == 4*G*KPL (no slot is out of range).
// The index data of batch b+1 is requested before batch b is computed.
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
    const uint64_t le = (lane == 63) ? ~0ull : ((2ull << lane) - 1ull);

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

        auto load_batch = [&](int bi) -> Batch {
            Batch b{-1, 0, 0, 0.f};
            const int pos = begin + (bi << 6) + lane;
            if (bi < b1 && pos < end) {
                const int gb = batch_base + bi;
                const int seg = segment_of(a, gb, pos, le);
                b.row = a.seg_row ? a.seg_row[seg] : seg;
                b.p = a.perm ? a.perm[pos] : pos;
                b.col = a.scol ? a.scol[pos] : a.col_ind[b.p];
                b.v = a.sval ? a.sval[pos] : (a.val ? a.val[b.p] : 1.0f);
            }
            return b;
        };

        int cur_row = -1;
        float4 w[KPL];
#pragma unroll
        for (int j = 0; j < KPL; ++j) w[j] = make_float4(0.f, 0.f, 0.f, 0.f);

        Batch nxt = load_batch(b0);
        for (int bi = b0; bi < b1; ++bi) {
            const Batch cur = nxt;
            nxt = load_batch(bi + 1);
            float acc[G];
#pragma unroll
            for (int i = 0; i < G; ++i) acc[i] = 0.f;

            const int row_first = group_bcast<G, 0>(cur.row);
            const int row_last = group_bcast<G, G - 1>(cur.row);
            if (row_first == row_last && row_last >= 0) {
                // all G nonzeros of this group lie in one row: no checks inside
                if (row_first != cur_row) {
                    cur_row = row_first;
                    const float4 *wr = W4 + (size_t)cur_row * K4;
#pragma unroll
                    for (int j = 0; j < KPL; ++j)
                        w[j] = (EXACT || slot[j] < K4) ? wr[slot[j]] : make_float4(0.f, 0.f, 0.f, 0.f);
                }
                [&]<int... I>(std::integer_sequence<int, I...>) {
                    ((void)[&] {
                        const int c_i = group_bcast<G, I>(cur.col);
                        const float4 *hr = LDS_TILE ? (lds_tile + (size_t)(c_i - tile_base) * K4)
                                                    : (H4 + (size_t)c_i * K4);
#pragma unroll
                        for (int j = 0; j < KPL; ++j)
                            if (EXACT || slot[j] < K4) acc[I] = dot4(w[j], hr[slot[j]], acc[I]);
                    }(), ...);
                }(std::make_integer_sequence<int, G>{});
            } else {
                [&]<int... I>(std::integer_sequence<int, I...>) {
                    ((void)[&] {
                        const int r_i = group_bcast<G, I>(cur.row);
                        const int c_i = group_bcast<G, I>(cur.col);
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
                                if (EXACT || slot[j] < K4) acc[I] = dot4(w[j], hr[slot[j]], acc[I]);
                        }
                    }(), ...);
                }(std::make_integer_sequence<int, G>{});
            }
            const float sum = transpose_reduce<G>(acc, l);
            if (cur.row >= 0) a.out[cur.p] = a.residual ? cur.v - sum : sum * cur.v;
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
        const uint64_t le = (lane == 63) ? ~0ull : ((2ull << lane) - 1ull);
        int row = -1, col = 0, p = 0;
        float v = 0.f;
        if (valid) {
            const int seg = segment_of(a, gb, pos, le);
            row = a.seg_row ? a.seg_row[seg] : seg;
            p = a.perm ? a.perm[pos] : pos;
            col = a.col_ind[p];
            v = a.val ? a.val[p] : 1.0f;
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
        if (valid) a.out[p] = a.residual ? v - sum : sum * v;
    }
}

}  // namespace

namespace sddmm {

// With H in LDS fewer lanes per nonzero pay (less cross-lane work per FMA);
// gathers from global memory prefer at least 8 lanes (128 contiguous bytes).
Variant pick_variant(int K, bool lds_tile)
{
    const int K4 = K / 4;
    if (lds_tile) {
        const int c4[][2] = {{4, 2}, {4, 4}, {4, 8}};
        for (auto &c : c4)
            if (c[0] * c[1] == K4) return {c[0], c[1], true};
    }
    const int cand[][2] = {{8, 1}, {8, 2}, {8, 3}, {8, 4}, {8, 6}, {8, 8}, {16, 6}, {16, 8}, {32, 6}, {32, 8}, {64, 6}, {64, 8}};
    for (auto &c : cand)
        if (c[0] * c[1] == K4) return {c[0], c[1], true};
    for (auto &c : cand)
        if (c[0] * c[1] >= K4) return {c[0], c[1], false};
    return {0, 0, false};  // K > 2048: generic kernel
}

template <bool LDS_TILE>
static KernelFn lookup(const Variant &v)
{
#define SDDMM_CASE(g, kpl)                                                              \
    if (v.G == g && v.KPL == kpl)                                                       \
        return v.exact ? (KernelFn)sddmm_stream_kernel<g, kpl, true, LDS_TILE>          \
                       : (KernelFn)sddmm_stream_kernel<g, kpl, false, LDS_TILE>;
    SDDMM_CASE(4, 2) SDDMM_CASE(4, 4) SDDMM_CASE(4, 8)
    SDDMM_CASE(8, 1) SDDMM_CASE(8, 2) SDDMM_CASE(8, 3) SDDMM_CASE(8, 4) SDDMM_CASE(8, 6) SDDMM_CASE(8, 8)
    SDDMM_CASE(16, 6) SDDMM_CASE(16, 8) SDDMM_CASE(32, 6) SDDMM_CASE(32, 8) SDDMM_CASE(64, 6) SDDMM_CASE(64, 8)
#undef SDDMM_CASE
    return nullptr;
}

__global__ void gather_values_kernel(const int32_t *__restrict__ perm, const float *__restrict__ src,
                                     float *__restrict__ dst, int64_t n)
{
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const int32_t p = perm[i];
        dst[i] = p >= 0 ? src[p] : 0.f;
    }
}

void launch_gather_values(const int32_t *perm, const float *src, float *dst, int64_t n, void *stream)
{
    if (n <= 0) return;
    const int blocks = (int)std::min<int64_t>((n + 255) / 256, 65536);
    hipLaunchKernelGGL(gather_values_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, perm, src, dst, n);
}

KernelFn stream_kernel(const Variant &v, bool lds_tile) { return lds_tile ? lookup<true>(v) : lookup<false>(v); }
KernelFn generic_kernel() { return (KernelFn)sddmm_generic_kernel; }

}  // namespace sddmm
