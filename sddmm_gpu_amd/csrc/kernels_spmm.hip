// The sparse-times-dense product Y = X H on a plan's column tiles, for gfx950 (MI355X):
// X has the pattern of S and one fp32 per nonzero (in sorted order), H is n_cols x K.
//
// Like the SDDMM's tile kernel a workgroup holds a column tile of H in LDS.  A (row, tile) run
// -- the nonzeros of one row inside one tile -- belongs to one group of 8 lanes from its first
// nonzero to its last: lane l keeps its 16 elements of the row of Y in registers and adds
// x[p] times its slice of the H row of every nonzero of the run, read from LDS.  No two groups
// ever add to the same row of Y: a run ends in one partial row, written once, in the order the
// runs are walked, and a second kernel adds the partial rows of every row of S (at most one per
// column tile).  No atomics, so the result has the same bits on every call.  The 8 groups of a
// wave walk 8 runs side by side ("bundle"); the planner sorts an item's runs by length, so a
// bundle's runs are about equally long.  Rows too short for the tiles gather their H rows from
// global memory, one group of lanes per row.
#include <hip/hip_runtime.h>
#include <utility>
#include "kernels.hpp"

using namespace sddmm;

namespace {

typedef float vec4f __attribute__((ext_vector_type(4)));

// The value that lane I of this lane's group of 8 holds, by two row broadcasts of the data-parallel
// primitives (one per half of a 16-lane row) and a select: vector-ALU work with no trip through the LDS
// pipe, which the H reads keep busy and whose latency would sit in front of every round.
template <int I>
__device__ __forceinline__ int from_group_lane(int v, bool upper_group)
{
    const int lo = __builtin_amdgcn_update_dpp(0, v, 0x150 + I, 0xf, 0xf, false);      // row_newbcast:I
    const int up = __builtin_amdgcn_update_dpp(0, v, 0x150 + I + 8, 0xf, 0xf, false);  // row_newbcast:I+8
    return upper_group ? up : lo;
}

// KPL float4 per lane: a K slice of 32 * KPL elements on groups of 8 lanes
template <int KPL, int NW>
__global__ __launch_bounds__(NW * 64)
void sddmm_spmm_tile_kernel(const SpmmArgs a)
{
    extern __shared__ float4 lds_tile[];
    constexpr int G = 8, K4 = G * KPL;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane & 7, g = lane >> 3;
    // the two groups of a 16-lane LDS phase read the halves of a 256-byte block in opposite order
    const int rot = KPL > 1 ? (g & 1) : 0;
    using lds_f4_ptr = const __attribute__((address_space(3))) vec4f *;
    const int lds_base = (int)(uint32_t)(uintptr_t)(lds_f4_ptr)reinterpret_cast<const vec4f *>(lds_tile);
    int piece[KPL];  // float4 index inside a row of this lane's j-th piece
#pragma unroll
    for (int j = 0; j < KPL; ++j) piece[j] = (j ^ rot) * G + l;
    // (its address is the row's + lane_e + 128 j for even j, + lane_o + 128 j for odd j: two adds per row)
    const int lane_e = lds_base + (l + rot * G) * 16, lane_o = lds_base + (l - rot * G) * 16;
    const int row_k4 = a.K >> 2;
    const float4 *__restrict__ H4 = reinterpret_cast<const float4 *>(a.H) + (a.k_off >> 2);
    float4 *__restrict__ part4 = reinterpret_cast<float4 *>(a.part);
    const int n_steps = (a.n_items - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    int cur_tile = -1;
    for (int step = 0; step < n_steps; ++step) {
        const WorkItem wi = a.items[blockIdx.x + step * gridDim.x];  // [begin, end): the item's bundles
        if (wi.end <= wi.begin) continue;
        if (wi.tile != cur_tile) {
            if (cur_tile >= 0) __syncthreads();
            cur_tile = wi.tile;
            const int tile_base = wi.tile * a.tile_x;
            const int rows = min(a.tile_x, a.n_cols - tile_base);
            const float4 *src = H4 + (size_t)tile_base * row_k4;
            const int n4 = rows * K4;
            for (int i = threadIdx.x; i < n4; i += NW * 64) {
                const int r = i / K4, q = i - r * K4;
                lds_tile[i] = src[(size_t)r * row_k4 + q];
            }
            __syncthreads();
        }
        // A wave takes the bundles wave, wave + NW, ... of the item.  While bundle b is walked, the headers of bundle
        // b + 2 NW and the first three rounds of bundle b + NW are requested; inside a bundle round r + 3 is requested
        // while round r is computed.  A round is 8 steps: lane l of a group fetches the column and the value of the
        // group's step 8 r + l, and the group's lanes take them from each other (from_group_lane).
        if (wi.begin + wave >= wi.end) continue;
        struct Hdr { int p0, len, off, n8; };
        auto header = [&](int b) -> Hdr {
            const int bc = min(b, wi.end - 1);  // (beyond the item: the last bundle again, never used)
            Hdr h;
            h.p0 = a.b_p0[bc * 8 + g]; h.len = a.b_len[bc * 8 + g];
            h.off = a.b_off[bc]; h.n8 = a.b_off[bc + 1] - h.off;
            return h;
        };
        struct Round { uint32_t c; float x; };
        auto fetch = [&](const Hdr &h, int r) -> Round {
            const int rc = min(r, h.n8 - 1);
            Round q;
            q.c = a.cols[((size_t)(h.off + rc) * 8 + g) * 8 + l];
            const int s = 8 * rc + l;
            const float xv = a.x[h.p0 + min(s, max(h.len, 1) - 1)];
            q.x = s < h.len ? xv : 0.f;
            return q;
        };
        Hdr h0 = header(wi.begin + wave), h1 = header(wi.begin + wave + NW);
        Round q0 = fetch(h0, 0), q1 = fetch(h0, 1), q2 = fetch(h0, 2);
        for (int b = wi.begin + wave; b < wi.end; b += NW) {
            const Hdr h2 = header(b + 2 * NW);
            Round n0 = fetch(h1, 0), n1 = fetch(h1, 1), n2 = fetch(h1, 2);
            const int n8 = __builtin_amdgcn_readfirstlane(h0.n8);
            float4 acc[KPL];
#pragma unroll
            for (int j = 0; j < KPL; ++j) acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            auto rd = [&](vec4f (&h)[KPL], int off) {
                const int addr_e = off + lane_e, addr_o = off + lane_o;
#pragma unroll
                for (int j = 0; j < KPL; ++j) h[j] = *(lds_f4_ptr)(uintptr_t)(uint32_t)(((j & 1) ? addr_o : addr_e) + j * 128);
            };
            for (int r = 0; r < n8; ++r) {
                const Round q3 = fetch(h0, r + 3);
                // the columns (as row offsets in the tile) and the values of the round's eight steps, taken from the
                // group's lanes
                int row_off[8];
                float xs[8];
                const int my_off = (int)q0.c * (K4 * 16), my_x = __float_as_int(q0.x);
                const bool upper = (lane & 8) != 0;
                [&]<int... I>(std::integer_sequence<int, I...>) {
                    ((row_off[I] = from_group_lane<I>(my_off, upper), xs[I] = __int_as_float(from_group_lane<I>(my_x, upper))), ...);
                }(std::make_integer_sequence<int, 8>{});
                // the H pieces of step i + 1 are requested before the arithmetic of step i
                vec4f hb[2][KPL];
                rd(hb[0], row_off[0]);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (i + 1 < 8) rd(hb[(i + 1) & 1], row_off[i + 1]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = 0; j < KPL; ++j) {
                        const vec4f h = hb[i & 1][j];
                        acc[j].x = fmaf(xs[i], h.x, acc[j].x); acc[j].y = fmaf(xs[i], h.y, acc[j].y);
                        acc[j].z = fmaf(xs[i], h.z, acc[j].z); acc[j].w = fmaf(xs[i], h.w, acc[j].w);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                q0 = q1; q1 = q2; q2 = q3;
            }
            if (h0.len > 0) {
                float4 *dst = part4 + ((size_t)b * 8 + g) * K4;
#pragma unroll
                for (int j = 0; j < KPL; ++j) dst[piece[j]] = acc[j];
            }
            h0 = h1; h1 = h2; q0 = n0; q1 = n1; q2 = n2;
        }
    }
}

// Y[row, slice] = sum of the row's partial rows: one wave per listed row, group g takes the partial
// rows g, g + 8, ... and the groups' sums are added across the wave.
template <int KPL>
__device__ __forceinline__ void spmm_sum_rows(const SpmmArgs &a, int64_t block)
{
    constexpr int G = 8, K4 = G * KPL;
    const int lane = threadIdx.x & 63, l = lane & 7, g = lane >> 3;
    const int64_t w = (block * 256 + threadIdx.x) >> 6;
    if (w >= a.n_sum_rows) return;
    const int b = a.row_part_ptr[w], e = a.row_part_ptr[w + 1];
    const float4 *__restrict__ part4 = reinterpret_cast<const float4 *>(a.part);
    float4 acc[KPL];
#pragma unroll
    for (int j = 0; j < KPL; ++j) acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = b + g; k < e; k += 8) {
        const float4 *src = part4 + (size_t)a.part_slot[k] * K4;
#pragma unroll
        for (int j = 0; j < KPL; ++j) {
            const float4 v = src[j * G + l];
            acc[j].x += v.x; acc[j].y += v.y; acc[j].z += v.z; acc[j].w += v.w;
        }
    }
#pragma unroll
    for (int off = 8; off < 64; off <<= 1) {
#pragma unroll
        for (int j = 0; j < KPL; ++j) {
            acc[j].x += __shfl_xor(acc[j].x, off); acc[j].y += __shfl_xor(acc[j].y, off);
            acc[j].z += __shfl_xor(acc[j].z, off); acc[j].w += __shfl_xor(acc[j].w, off);
        }
    }
    if (g == 0) {
        float4 *y = reinterpret_cast<float4 *>(a.Y) + (size_t)a.sum_rows[w] * (a.K >> 2) + (a.k_off >> 2);
#pragma unroll
        for (int j = 0; j < KPL; ++j) y[j * G + l] = acc[j];
    }
}

// The rows outside the tiles (short ones, and rows without entries, which become 0): one group of 8
// lanes per row, H rows gathered from global memory, four nonzeros in flight per step; the planner lists
// the rows longest first, so that the eight rows of a wave are about equally long.
template <int KPL>
__device__ __forceinline__ void spmm_gather_rows(const SpmmArgs &a, int64_t block)
{
    constexpr int G = 8;
    const int lane = threadIdx.x & 63, l = lane & 7;
    const int64_t grp = (block * 256 + threadIdx.x) >> 3;
    if (grp >= a.n_gather_rows) return;
    const int row = a.gather_rows[grp];
    const int b = a.row_ptr[row], e = a.row_ptr[row + 1];
    const int row_k4 = a.K >> 2;
    const float4 *__restrict__ H4 = reinterpret_cast<const float4 *>(a.H) + (a.k_off >> 2) + l;
    float4 acc[KPL];
#pragma unroll
    for (int j = 0; j < KPL; ++j) acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    auto add = [&](const float4 *hr, float xs) {
#pragma unroll
        for (int j = 0; j < KPL; ++j) {
            const float4 h = hr[j * G];
            acc[j].x = fmaf(xs, h.x, acc[j].x); acc[j].y = fmaf(xs, h.y, acc[j].y);
            acc[j].z = fmaf(xs, h.z, acc[j].z); acc[j].w = fmaf(xs, h.w, acc[j].w);
        }
    };
    int p = b;
    for (; p + 3 < e; p += 4) {
        int cc[4]; float xx[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) { cc[i] = a.col_ind[p + i]; xx[i] = a.x[p + i]; }
        float4 hh[4][KPL];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < KPL; ++j) hh[i][j] = H4[(size_t)cc[i] * row_k4 + j * G];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < KPL; ++j) {
                acc[j].x = fmaf(xx[i], hh[i][j].x, acc[j].x); acc[j].y = fmaf(xx[i], hh[i][j].y, acc[j].y);
                acc[j].z = fmaf(xx[i], hh[i][j].z, acc[j].z); acc[j].w = fmaf(xx[i], hh[i][j].w, acc[j].w);
            }
    }
    for (; p < e; ++p) add(H4 + (size_t)a.col_ind[p] * row_k4, a.x[p]);
    float4 *y = reinterpret_cast<float4 *>(a.Y) + (size_t)row * row_k4 + (a.k_off >> 2) + l;
#pragma unroll
    for (int j = 0; j < KPL; ++j) y[j * G] = acc[j];
}

// Second kernel of a slice: the sums of the partial rows (a stream through memory) and the rows outside
// the tiles (gathers from L2) side by side, sum_blocks and gather_blocks workgroups of each spread evenly
// over the grid, so that the two kinds of traffic overlap.
template <int KPL>
__global__ __launch_bounds__(256)
void sddmm_spmm_rows_kernel(const SpmmArgs a, int64_t sum_blocks, int64_t gather_blocks)
{
    const int64_t i = blockIdx.x, n = sum_blocks + gather_blocks;
    const int64_t sums_before = i * sum_blocks / n;  // (of the workgroups 0 .. i - 1)
    if ((i + 1) * sum_blocks / n > sums_before) spmm_sum_rows<KPL>(a, sums_before);
    else spmm_gather_rows<KPL>(a, i - sums_before);
}

}  // namespace

namespace sddmm {

bool spmm_tile_supported(int k_slice)
{
    return k_slice == 32 || k_slice == 64 || k_slice == 128;
}

int spmm_tile_set_lds(int k_slice, int nwaves, int lds_bytes)
{
    const void *fn = nullptr;
#define SDDMM_SPMM_FN(kpl) (nwaves == 12 ? (const void *)sddmm_spmm_tile_kernel<kpl, 12> : (const void *)sddmm_spmm_tile_kernel<kpl, 16>)
    if (k_slice == 128) fn = SDDMM_SPMM_FN(4);
    else if (k_slice == 64) fn = SDDMM_SPMM_FN(2);
    else if (k_slice == 32) fn = SDDMM_SPMM_FN(1);
#undef SDDMM_SPMM_FN
    if (!fn) return 1;
    return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) == hipSuccess ? 0 : 2;
}

// one K slice of the product: the tile kernel over the bundles, the sum of the partial rows, the gathered rows
void launch_spmm_slice(const SpmmArgs &a, int k_slice, int nwaves, int grid, int lds_bytes, void *stream)
{
    hipStream_t st = (hipStream_t)stream;
    const unsigned sum_grid = (unsigned)((a.n_sum_rows + 3) / 4);
    const unsigned rows_grid = (unsigned)((a.n_gather_rows + 31) / 32);
#define SDDMM_SPMM_LAUNCH(kpl)                                                                                         \
    do {                                                                                                               \
        if (a.n_items > 0) {                                                                                           \
            if (nwaves == 12) hipLaunchKernelGGL((sddmm_spmm_tile_kernel<kpl, 12>), dim3((unsigned)grid), dim3(12 * 64), (size_t)lds_bytes, st, a); \
            else hipLaunchKernelGGL((sddmm_spmm_tile_kernel<kpl, 16>), dim3((unsigned)grid), dim3(16 * 64), (size_t)lds_bytes, st, a);              \
        }                                                                                                              \
        if (sum_grid + rows_grid > 0)                                                                                  \
            hipLaunchKernelGGL((sddmm_spmm_rows_kernel<kpl>), dim3(sum_grid + rows_grid), dim3(256), 0, st, a, (int64_t)sum_grid, (int64_t)rows_grid); \
    } while (0)
    if (k_slice == 128) SDDMM_SPMM_LAUNCH(4);
    else if (k_slice == 64) SDDMM_SPMM_LAUNCH(2);
    else if (k_slice == 32) SDDMM_SPMM_LAUNCH(1);
#undef SDDMM_SPMM_LAUNCH
}

}  // namespace sddmm
