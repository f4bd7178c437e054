// The two forms that surround an SDDMM in its machine-learning uses, for gfx950 (MI355X):
// the row-wise softmax of the sampled products (attention scores restricted to the pattern
// of S) and the sparse-times-dense product that consumes them, Y = softmax(S .* W H^T) H.
// Both work on the sorted S directly (CSR pointers + one fp32 per nonzero), so they follow a
// plan's sddmm_execute on the same stream without any re-ordering.
#include <hip/hip_runtime.h>
#include <mutex>
#include "internal.hpp"

using namespace sddmm;

namespace {

// Row softmax.  Every row is worked on whole, in registers, by as many lanes as its length asks for, so
// that an entry is read once and written once whatever the rows' lengths (a matrix may hold a few rows of
// a million entries next to millions of rows of ten, so the work is cut by entries, not by rows):
//   short rows (up to kSmChunk entries) are grouped into chunks of consecutive whole rows: chunk c
//        starts with the row that holds entry c * kSmChunk and ends before the row that holds entry
//        (c + 1) * kSmChunk.  A wave takes a chunk, 64 of its rows at a time: a lane per row of up to 8
//        entries, then groups of 8 lanes (up to 96), of 32 lanes (up to 512), the whole wave (up to 1024
//        in registers, beyond that in two walks over the row).
//   long rows (up to kSmLongMax entries) belong to no chunk: a workgroup each (the recommender shape
//        keeps 56 % of its entries in rows of more than 4096).
//   huge rows (beyond that) are cut at the multiples of kSmChunk: a workgroup takes a piece, stores it
//        as exp(x - m) with the piece's own maximum m and leaves (m, sum) in a record of the chunk; a last
//        kernel merges the records of each huge row and scales its pieces.
// Three kernels: the first lays the chunks out (one thread per chunk); the second takes the short rows
// with two thirds of its workgroups and the long rows and pieces with the others; the last works from two
// lists that the second makes.  All read the number of entries from row_ptr[n_rows] on the device and walk
// the chunks with a grid-sized stride.  No LDS staging: a
// row's loads are all in flight together, and 16 waves per compute unit hide their latency.
constexpr int kSmChunk = 4096;
constexpr int kSmBlock = 256;
constexpr int64_t kSmMaxChunks = ((int64_t)1 << 31) / kSmChunk;
constexpr int kSmLongQ = 16;                             // float4 per thread of the long-row kernel
constexpr int kSmLongMax = kSmLongQ * 4 * kSmBlock - 8;  // (less what a misaligned start costs)
constexpr int kSmListRows = 1 << 30, kSmListHuge = 1 << 29, kSmListChunk = kSmListHuge - 1;  // an item of the last kernel's list: flags | chunk
constexpr int kSmOwnBatches = 32;                       // batches of 64 rows that a chunk's own wave takes at least
constexpr int kSmByLane = 8, kSmBy8 = 96, kSmBy32 = 512, kSmByWave16 = 1024;  // row lengths up to which a lane / 8 lanes / 32 lanes / the wave with 16 entries per lane work on a row

__device__ __forceinline__ int softmax_row_class(int64_t len) { return len <= kSmChunk ? 0 : len <= kSmLongMax ? 1 : 2; }

// (m, sum) of the pieces of huge rows: [2c] the row that began before chunk c, [2c + 1] the row that ends
// after it; and the layout of each chunk: first entry, end, first row, last row.  The kernels take both
// arrays as arguments: a caller's workspace (sddmm_execute_ws), or these file-scope arrays, 8 + 8 + 2 MiB per
// device, held until the process ends -- softmax calls without a workspace that overlap in time on one
// device share them and must not (calls on one stream never do).
static __device__ __align__(256) float2 g_softmax_rec_store[2 * kSmMaxChunks];
static __device__ __align__(256) int4 g_softmax_rows_store[kSmMaxChunks];
// the last kernel's work, 2 MiB: [0] and [1] the lengths of two lists of chunks (with flags), one from [2] upwards, the
// other from [n_chunks + 1] downwards (a chunk is in one of them at most)
static __device__ __align__(256) int32_t g_softmax_list_store[kSmMaxChunks + 64];

// First kernel: the layout, one thread per chunk (a binary search of row_ptr whose loads the other
// threads' searches hide).  With r the row that holds entry c * kSmChunk, chunk c begins at r's first
// entry (r short), after r's last (r long; the chunk may come out empty) or at entry c * kSmChunk itself
// (r huge); it ends where chunk c + 1 would begin if that row were short (so a long row that starts
// past the chunk's rows is left out) or at the multiple (huge).  The row of chunk c + 1 is the next
// thread's search: a workgroup of 256 threads lays out 255 chunks (the kernel is bound by the number of
// its scattered loads).
__global__ __launch_bounds__(256)
void sddmm_row_softmax_rows_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, int4 *__restrict__ g_softmax_rows,
                                   int32_t *__restrict__ g_softmax_list)
{
    __shared__ int row_of[256], begin_of[256], end_of[256];  // the row that holds a chunk's first entry, and its extent
    if (blockIdx.x == 0 && threadIdx.x < 2) g_softmax_list[threadIdx.x] = 0;  // (the second kernel counts in them)
    const int64_t nnz = row_ptr[n_rows];
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    for (int64_t base = (int64_t)blockIdx.x * 255; base < n_chunks; base += (int64_t)gridDim.x * 255) {
        const int64_t c = base + threadIdx.x, p0 = c * kSmChunk;
        int64_t lo0 = 0, b0 = 0, e0 = 0;
        if (c < n_chunks) {
            int64_t hi0 = n_rows - 1;  // first row whose end lies beyond p0
            while (lo0 < hi0) {
                const int64_t mid = (lo0 + hi0) >> 1;
                if (row_ptr[mid + 1] <= p0) lo0 = mid + 1; else hi0 = mid;
            }
            b0 = row_ptr[lo0];
            e0 = row_ptr[lo0 + 1];
        }
        __syncthreads();  // (the round before has read its neighbours' rows)
        row_of[threadIdx.x] = (int)lo0; begin_of[threadIdx.x] = (int)b0; end_of[threadIdx.x] = (int)e0;
        __syncthreads();
        if (c >= n_chunks || threadIdx.x == 255) continue;
        int4 lay;
        const int k0 = softmax_row_class(e0 - b0);
        lay.x = (int)(k0 == 0 ? b0 : k0 == 1 ? e0 : p0);
        lay.z = (int)(k0 == 1 ? lo0 + 1 : lo0);
        if (p0 + kSmChunk >= nnz) {
            lay.y = (int)nnz;
            lay.w = (int)(n_rows - 1);
        } else {  // (chunk c + 1 exists: its first entry p0 + kSmChunk is an entry)
            const int64_t lo1 = row_of[threadIdx.x + 1], b1 = begin_of[threadIdx.x + 1], e1 = end_of[threadIdx.x + 1];
            const int k1 = softmax_row_class(e1 - b1);
            lay.y = (int)(k1 == 2 ? p0 + kSmChunk : b1);
            lay.w = (int)(k1 == 2 ? lo1 : lo1 - 1);
        }
        g_softmax_rows[c] = lay;
    }
}

// exp(x) for x <= 0 in six instructions: 2^t with t = x log2(e) rounded, times 1 + (what the rounding of t
// and of log2(e) left out) ln 2.  About one ulp; the library routine costs four times as much, and these
// passes would be bound by it.
__device__ __forceinline__ float exp_nonpositive(float x)
{
    const float l2e = 1.44269502e+0f, l2e_lo = 1.92596299e-8f;
    const float t = x * l2e;
    const float r = fmaf(x, l2e_lo, fmaf(x, l2e, -t));
    const float e = __builtin_amdgcn_exp2f(t);
    return fmaf(e, r * 0.693147182f, e);
}

template <int GW>
__device__ __forceinline__ float group_max(float v)
{
#pragma unroll
    for (int off = GW / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
}
template <int GW>
__device__ __forceinline__ float group_sum(float v)
{
#pragma unroll
    for (int off = GW / 2; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// One whole row of len entries at xr / outr by a group of GW lanes (GW = 1: the lane alone), R entries
// per lane, all of them requested before the first is used.  Every lane of the wave runs through this
// (the lane exchanges must not sit under a branch); `mine` says whether the lane's group has a row.
template <int GW, int R>
__device__ __forceinline__ void softmax_row_by_group(const float *xr, float *outr, int len, bool mine)
{
    const int gl = threadIdx.x & (GW - 1);
    if (!mine) len = 0;
    float v[R];
#pragma unroll
    for (int k = 0; k < R; ++k) v[k] = gl + k * GW < len ? xr[gl + k * GW] : -INFINITY;
    float m = v[0];
#pragma unroll
    for (int k = 1; k < R; ++k) m = fmaxf(m, v[k]);
    m = group_max<GW>(m);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < R; ++k) {
        v[k] = gl + k * GW < len ? exp_nonpositive(v[k] - m) : 0.f;
        sum += v[k];
    }
    sum = group_sum<GW>(sum);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int k = 0; k < R; ++k) if (gl + k * GW < len) outr[gl + k * GW] = v[k] * inv;
}

// The same for a row too long for the registers of its group: a first walk, R entries per lane at a time,
// keeps a running maximum and the sum of exponentials relative to it; a second walk (the row is in the
// caches by then) writes exp(x - max) / sum.
template <int GW, int R>
__device__ __forceinline__ void softmax_row_in_two_walks(const float *xr, float *outr, int len)
{
    const int gl = threadIdx.x & (GW - 1);
    float m = -INFINITY, sum = 0.f;
    for (int base = gl; base < len; base += GW * R) {
        float v[R];
#pragma unroll
        for (int k = 0; k < R; ++k) v[k] = base + k * GW < len ? xr[base + k * GW] : -INFINITY;
        float mn = m;
#pragma unroll
        for (int k = 0; k < R; ++k) mn = fmaxf(mn, v[k]);
        sum = m == -INFINITY ? 0.f : sum * exp_nonpositive(m - mn);
#pragma unroll
        for (int k = 0; k < R; ++k) sum += base + k * GW < len ? exp_nonpositive(v[k] - mn) : 0.f;
        m = mn;
    }
    const float all = group_max<GW>(m);
    sum = m == -INFINITY ? 0.f : sum * exp_nonpositive(m - all);
    sum = group_sum<GW>(sum);
    const float inv = 1.0f / sum;
    for (int base = gl; base < len; base += GW * R) {
        float v[R];
#pragma unroll
        for (int k = 0; k < R; ++k) v[k] = base + k * GW < len ? xr[base + k * GW] : -INFINITY;
#pragma unroll
        for (int k = 0; k < R; ++k) if (base + k * GW < len) outr[base + k * GW] = exp_nonpositive(v[k] - all) * inv;
    }
}

// How many batches of 64 rows the wave of a chunk takes itself.  A chunk with more rows than that (4096
// entries spread over many rows: mostly empty ones) would hold its wave long after the others are done:
// its further batches go to the whole machine (the last kernel), so no wave takes much more than twice the
// average.
__device__ __forceinline__ int64_t softmax_own_batches(int64_t n_rows, int64_t n_chunks)
{
    return max((int64_t)kSmOwnBatches, 2 * (n_rows / (64 * max(n_chunks, (int64_t)1)) + 1));
}

// The short rows among the 64 rows from w0 (up to row `last`), by one wave.
__device__ __forceinline__ void softmax_row_batch(const int32_t *__restrict__ row_ptr, const float *x, float *out, int64_t w0,
                                                  int64_t last, int lane)
{
        {
            const int64_t r = w0 + lane;
            int64_t rb = 0;
            int len = 0;
            if (r <= last) {
                rb = row_ptr[r];
                const int64_t l = (int64_t)row_ptr[r + 1] - rb;
                len = l <= kSmChunk ? (int)l : 0;  // (a huge row at either end of the chunk is not this kernel's)
            }
            // a lane per row
            if (__ballot(len >= 1 && len <= kSmByLane)) softmax_row_by_group<1, kSmByLane>(x + rb, out + rb, len, len <= kSmByLane);
            // groups of 8 lanes: eight rows at a time
            uint64_t todo = __ballot(len > kSmByLane && len <= kSmBy8);
            while (todo) {
                int src = -1;  // the lane that holds the row of this lane's group
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    const int b = todo ? __builtin_ctzll(todo) : -1;
                    if (todo) todo &= todo - 1;
                    if ((lane >> 3) == g) src = b;
                }
                const int64_t gb = __shfl(rb, src < 0 ? lane : src);
                const int gn = __shfl(len, src < 0 ? lane : src);
                softmax_row_by_group<8, kSmBy8 / 8>(x + gb, out + gb, gn, src >= 0);
            }
            // groups of 32 lanes: two rows at a time
            todo = __ballot(len > kSmBy8 && len <= kSmBy32);
            while (todo) {
                int src = -1;
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    const int b = todo ? __builtin_ctzll(todo) : -1;
                    if (todo) todo &= todo - 1;
                    if ((lane >> 5) == g) src = b;
                }
                const int64_t gb = __shfl(rb, src < 0 ? lane : src);
                const int gn = __shfl(len, src < 0 ? lane : src);
                softmax_row_by_group<32, kSmBy32 / 32>(x + gb, out + gb, gn, src >= 0);
            }
            // the whole wave: row by row
            todo = __ballot(len > kSmBy32);
            while (todo) {
                const int b = __builtin_ctzll(todo);
                todo &= todo - 1;
                const int64_t gb = __shfl(rb, b);
                const int gn = __shfl(len, b);
                if (gn <= kSmByWave16) softmax_row_by_group<64, kSmByWave16 / 64>(x + gb, out + gb, gn, true);
                else softmax_row_in_two_walks<64, kSmByWave16 / 64>(x + gb, out + gb, gn);
            }
        }
}

// The short rows, a wave per chunk; workgroup `group` of `n_groups`.
__device__ __forceinline__ void softmax_short_rows(const int32_t *__restrict__ row_ptr, int64_t n_rows, const float *x, float *out,
                                                   const int4 *__restrict__ g_softmax_rows, int64_t group, int64_t n_groups)
{
    const int lane = threadIdx.x & 63;
    const int64_t nnz = row_ptr[n_rows];
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    const int64_t n_waves = n_groups * (kSmBlock / 64);
    const int64_t own = softmax_own_batches(n_rows, n_chunks);
    for (int64_t c = group * (kSmBlock / 64) + (threadIdx.x >> 6); c < n_chunks; c += n_waves) {
        const int4 lay = g_softmax_rows[c];
        if (lay.x >= lay.y) continue;
        const int64_t last = min((int64_t)lay.w, (int64_t)lay.z + 64 * own - 1);
        for (int64_t w0 = lay.z; w0 <= last; w0 += 64) softmax_row_batch(row_ptr, x, out, w0, last, lane);
    }
}

// One long row, or one piece of a huge row, [rb, re) by a workgroup of kSmBlock threads, held in registers
// (4 * NQ floats per thread): read once, written once.  x 16-byte aligned: float4 pieces counted from the
// aligned address below the first entry (entries outside are masked); otherwise single entries, strided.
// rec = NULL: a whole row, normalised; otherwise a piece, stored as exp(x - max) with (max, sum) in *rec.
template <int NQ>
__device__ __forceinline__ void softmax_long_row(const float *x, float *out, int64_t rb, int64_t re, int64_t nnz, bool vec_in,
                                                 bool vec_out, float *red, float2 *rec)
{
    constexpr int NW = kSmBlock / 64;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    // (offsets relative to the aligned address below the row's start fit 32 bits)
    const int64_t a0 = vec_in ? (rb & ~(int64_t)3) : rb;
    const float *xr = x + a0;
    float *outr = out + a0;
    const int head = (int)(rb - a0), end = (int)(re - a0);
    const int lim = (int)min(nnz - a0, (int64_t)INT32_MAX);  // entries of the array from a0 on
    float f[4 * NQ];
    if (vec_in) {
#pragma unroll
        for (int k = 0; k < NQ; ++k) {
            const int p = 4 * (t + k * kSmBlock);
            float4 v = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
            if (p < end) {
                if (p + 3 < lim) {
                    v = *reinterpret_cast<const float4 *>(xr + p);
                } else {
                    v.x = xr[p];
                    if (p + 1 < lim) v.y = xr[p + 1];
                    if (p + 2 < lim) v.z = xr[p + 2];
                }
            }
            f[4 * k + 0] = (p + 0 >= head && p + 0 < end) ? v.x : -INFINITY;
            f[4 * k + 1] = (p + 1 >= head && p + 1 < end) ? v.y : -INFINITY;
            f[4 * k + 2] = (p + 2 >= head && p + 2 < end) ? v.z : -INFINITY;
            f[4 * k + 3] = (p + 3 >= head && p + 3 < end) ? v.w : -INFINITY;
        }
    } else {
#pragma unroll
        for (int k = 0; k < 4 * NQ; ++k) {
            const int p = t + k * kSmBlock;
            f[k] = p < end ? xr[p] : -INFINITY;
        }
    }
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < 4 * NQ; ++k) m = fmaxf(m, f[k]);
    m = group_max<64>(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < NW; ++w) m = fmaxf(m, red[w]);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < 4 * NQ; ++k) {
        f[k] = f[k] == -INFINITY ? 0.f : exp_nonpositive(f[k] - m);
        sum += f[k];
    }
    sum = group_sum<64>(sum);
    if (lane == 0) red[NW + wave] = sum;
    __syncthreads();
    sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += red[NW + w];
    const float inv = rec ? 1.0f : 1.0f / sum;
    if (rec && t == 0) *rec = make_float2(m, sum);
    if (vec_in) {
#pragma unroll
        for (int k = 0; k < NQ; ++k) {
            const int p = 4 * (t + k * kSmBlock);
            if (p >= end) continue;
            if (vec_out && p >= head && p + 4 <= end) {
                *reinterpret_cast<float4 *>(outr + p) = make_float4(f[4 * k] * inv, f[4 * k + 1] * inv, f[4 * k + 2] * inv, f[4 * k + 3] * inv);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) if (p + j >= head && p + j < end) outr[p + j] = f[4 * k + j] * inv;
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < 4 * NQ; ++k) {
            const int p = t + k * kSmBlock;
            if (p < end) outr[p] = f[k] * inv;
        }
    }
    // (the next row writes its maxima after this row's second barrier and its sums after its own first: no barrier needed here)
}

// The long rows and the pieces of huge rows; workgroup `group` of `n_groups`.  A long row holds the multiple of kSmChunk
// that follows its first entry, so it is the row after the last row of the chunk whose window
// [c * kSmChunk, (c + 1) * kSmChunk) it starts in; a huge row is the first or the last row of every chunk
// it touches.  Workgroup b looks at the chunks b, b + n_groups, ...: first at many of them at once, a thread
// per chunk (a few dependent loads each, which a walk chunk by chunk would pay for one after the other),
// what it finds collected in a list; then the list item by item.
__device__ __forceinline__ void softmax_long_rows(const int32_t *__restrict__ row_ptr, int64_t n_rows, const float *x, float *out,
                                                  float2 *g_softmax_rec, const int4 *__restrict__ g_softmax_rows, int32_t *g_softmax_list,
                                                  int64_t group, int64_t n_groups)
{
    __shared__ float red[2 * kSmBlock / 64];
    __shared__ int4 todo[3 * kSmBlock];  // first entry, end, record (-1: a whole row)
    __shared__ int n_todo;
    const int64_t nnz = row_ptr[n_rows];
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    const bool vec_in = (reinterpret_cast<uintptr_t>(x) & 15u) == 0, vec_out = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    const int64_t own = softmax_own_batches(n_rows, n_chunks);
    for (int64_t base = group; base < n_chunks; base += n_groups * kSmBlock) {
        __syncthreads();  // the list of the round before has been worked off
        if (threadIdx.x == 0) n_todo = 0;
        __syncthreads();
        const int64_t c = base + (int64_t)threadIdx.x * n_groups;
        int item = 0;  // this chunk's item of the last kernel's lists, if it has one
        if (c < n_chunks) {
            const int4 lay = g_softmax_rows[c];
            const int64_t r = (int64_t)lay.w + 1;
            if (r < n_rows) {
                const int64_t rb = row_ptr[r], re = row_ptr[r + 1];
                if (rb >= c * kSmChunk && rb < (c + 1) * kSmChunk && softmax_row_class(re - rb) == 1)
                    todo[atomicAdd(&n_todo, 1)] = make_int4((int)rb, (int)re, -1, 0);
            }
            if (lay.x < lay.y) {
                const int64_t c0 = lay.x, c1 = lay.y, r0 = lay.z, r1 = lay.w;
                // for the last kernel: more rows than the chunk's own wave takes; pieces of huge rows
                item = (r1 - r0) / 64 + 1 > own ? kSmListRows : 0;
                const int64_t b0 = row_ptr[r0], e0 = row_ptr[r0 + 1];
                if (softmax_row_class(e0 - b0) == 2) {
                    todo[atomicAdd(&n_todo, 1)] = make_int4((int)max(b0, c0), (int)min(e0, c1), (int)(2 * c + (b0 < c0 ? 0 : 1)), 0);
                    item |= kSmListHuge;
                }
                if (r1 != r0) {
                    const int64_t b1 = row_ptr[r1], e1 = row_ptr[r1 + 1];
                    if (softmax_row_class(e1 - b1) == 2) {
                        todo[atomicAdd(&n_todo, 1)] = make_int4((int)max(b1, c0), (int)min(e1, c1), (int)(2 * c + 1), 0);
                        item |= kSmListHuge;
                    }
                }
            }
        }
        // Chunks with rows left go to the list that all workgroups will read, chunks with pieces of huge rows
        // only to the one of which a workgroup reads its share; one addition to a list's length per wave.
        {
            const int lane = threadIdx.x & 63;
            const bool rows_left = item & kSmListRows;
            const uint64_t front = __ballot(rows_left), back = __ballot(item && !rows_left), below = ((uint64_t)1 << lane) - 1;
            if (front) {
                const int first = __builtin_ctzll(front);
                int at = 0;
                if (lane == first) at = atomicAdd(&g_softmax_list[0], __builtin_popcountll(front));
                at = __shfl(at, first);
                if (rows_left) g_softmax_list[2 + at + __builtin_popcountll(front & below)] = item | (int)c;
            }
            if (back) {
                const int first = __builtin_ctzll(back);
                int at = 0;
                if (lane == first) at = atomicAdd(&g_softmax_list[1], __builtin_popcountll(back));
                at = __shfl(at, first);
                if (item && !rows_left) g_softmax_list[n_chunks + 1 - at - __builtin_popcountll(back & below)] = item | (int)c;
            }
        }
        __syncthreads();
        const int n = n_todo;
        for (int q = 0; q < n; ++q) {
            const int4 w = todo[q];
            const int64_t rb = w.x, re = w.y;
            float2 *rec = w.z < 0 ? nullptr : &g_softmax_rec[w.z];
            if (re - rb <= 8 * 4 * kSmBlock - 8) softmax_long_row<8>(x, out, rb, re, nnz, vec_in, vec_out, red, rec);
            else softmax_long_row<kSmLongQ>(x, out, rb, re, nnz, vec_in, vec_out, red, rec);
        }
    }
}

// Second kernel: every third workgroup takes the long rows, the others the short ones; the two kinds of
// work fill each other's gaps (a long row's workgroup loads, then reduces, then stores).
__global__ __launch_bounds__(kSmBlock, 4)  // (four waves per SIMD: four long rows in flight per compute unit)
void sddmm_row_softmax_main_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, const float *x, float *out,
                                   float2 *g_softmax_rec, const int4 *__restrict__ g_softmax_rows, int32_t *g_softmax_list)
{
    // (a third for the long rows: measured against a half and a quarter on a recommender and an R-MAT pattern)
    constexpr int every = 3;
    const int64_t n_long = (gridDim.x + every - 1) / every, mine = blockIdx.x / every;
    if (blockIdx.x % every == 0) softmax_long_rows(row_ptr, n_rows, x, out, g_softmax_rec, g_softmax_rows, g_softmax_list, mine, n_long);
    else softmax_short_rows(row_ptr, n_rows, x, out, g_softmax_rows, blockIdx.x - mine - 1, gridDim.x - n_long);
}

// (m, sum) of the huge row [rb, re) from the records of the chunks it spans: the last-slot record of its
// first chunk, the first-slot records of the others; every wave of the workgroup computes the same pair.
__device__ __forceinline__ float2 merged_record(const float2 *__restrict__ g_softmax_rec, int64_t rb, int64_t re)
{
    const int lane = threadIdx.x & 63;
    const int64_t ca = rb / kSmChunk, cb = (re - 1) / kSmChunk;
    float m = -INFINITY, s = 0.f;
    for (int64_t k = ca + lane; k <= cb; k += 64) {
        const float2 rec = g_softmax_rec[2 * k + (k == ca ? 1 : 0)];
        const float mn = fmaxf(m, rec.x);
        s = s * expf(m - mn) + rec.y * expf(rec.x - mn);  // (exp(-inf - finite) = 0 for the first record)
        m = mn;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float m2 = __shfl_xor(m, off), s2 = __shfl_xor(s, off);
        const float mn = fmaxf(m, m2);
        // (a lane without records holds (-inf, 0): its term must vanish without producing inf - inf)
        const float t1 = m == -INFINITY ? 0.f : s * expf(m - mn), t2 = m2 == -INFINITY ? 0.f : s2 * expf(m2 - mn);
        s = t1 + t2;
        m = mn;
    }
    return make_float2(m, s);
}

// out[b..e) *= f by the whole workgroup, eight entries per thread in flight
__device__ __forceinline__ void scale_range(float *out, int64_t b, int64_t e, float f)
{
    for (int64_t i0 = b + threadIdx.x; i0 < e; i0 += 8 * kSmBlock) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = i0 + u * kSmBlock < e ? out[i0 + u * kSmBlock] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) if (i0 + u * kSmBlock < e) out[i0 + u * kSmBlock] = v[u] * f;
    }
}

// The pieces of huge rows in chunk c are scaled to the whole row's maximum and sum, by a workgroup.  A chunk
// holds at most two of them: at its beginning (the row came from the chunk before, or fills this one and
// goes on) and at its end.
__device__ __forceinline__ void softmax_merge_chunk(const int32_t *__restrict__ row_ptr, float *out, const float2 *__restrict__ g_softmax_rec,
                                                    const int4 *__restrict__ g_softmax_rows, int64_t c)
{
    const int4 lay = g_softmax_rows[c];
    const int64_t c0 = lay.x, c1 = lay.y, r0 = lay.z, r1 = lay.w;
    const int64_t b0 = row_ptr[r0], e0 = row_ptr[r0 + 1], b1 = row_ptr[r1], e1 = row_ptr[r1 + 1];
    if (softmax_row_class(e0 - b0) == 2 && (b0 < c0 || e0 > c1)) {  // a huge row begins the chunk
        const float2 all = merged_record(g_softmax_rec, b0, e0);
        const float2 mine = g_softmax_rec[2 * c + (b0 < c0 ? 0 : 1)];
        const float f = expf(mine.x - all.x) / all.y;
        const int64_t pb = max(b0, c0), pe = min(e0, c1);
        scale_range(out, pb, pe, f);
    }
    if (r1 != r0 && softmax_row_class(e1 - b1) == 2 && e1 > c1) {  // another one begins inside the chunk and ends after it
        const float2 all = merged_record(g_softmax_rec, b1, e1);
        const float2 mine = g_softmax_rec[2 * c + 1];
        const float f = expf(mine.x - all.x) / all.y;
        scale_range(out, b1, c1, f);
    }
}

// Last kernel, over the two lists that the second kernel made.
//  - The chunks whose own wave left batches of rows.  Every workgroup reads that whole list, kSmBlock items
//    at a time (on most matrices it is empty), and takes its share: a chunk's further batches in parts of
//    kSmPart (one or two per wave of a workgroup), part p of list item i with the workgroup (i + p) mod
//    gridDim.x; if the chunk holds pieces of huge rows too, workgroup i mod gridDim.x merges them.
//  - The other chunks with pieces of huge rows: item i with the workgroup i mod gridDim.x.
constexpr int kSmPart = 2 * (kSmBlock / 64);

__global__ __launch_bounds__(kSmBlock)
void sddmm_row_softmax_merge_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, const float *x, float *out,
                                    const float2 *__restrict__ g_softmax_rec, const int4 *__restrict__ g_softmax_rows,
                                    const int32_t *__restrict__ g_softmax_list)
{
    __shared__ int64_t todo_first[2 * kSmBlock];  // first row of this workgroup's first part of a chunk; or -1 - chunk: its huge rows' pieces
    __shared__ int todo_last[2 * kSmBlock];       // the chunk's last row
    __shared__ int n_todo;
    const int n_list = g_softmax_list[0], n_huge = g_softmax_list[1];
    if (n_list <= 0 && n_huge <= 0) return;
    const int64_t nnz = row_ptr[n_rows];
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t own = softmax_own_batches(n_rows, n_chunks), G = gridDim.x;
    for (int base = 0; base < n_list; base += kSmBlock) {
        __syncthreads();  // the list of the round before has been worked off
        if (threadIdx.x == 0) n_todo = 0;
        __syncthreads();
        const int i = base + (int)threadIdx.x;
        if (i < n_list) {
            const int item = g_softmax_list[2 + i], c = item & kSmListChunk;
            const int4 lay = g_softmax_rows[c];
            const int64_t first = (int64_t)lay.z + 64 * own;  // (<= lay.w: that is why the chunk is in this list)
            const int64_t parts = (((int64_t)lay.w - first) / 64 + kSmPart) / kSmPart;
            const int64_t p0 = (((int64_t)blockIdx.x - i) % G + G) % G;
            if (p0 < parts) {
                const int k = atomicAdd(&n_todo, 1);
                todo_first[k] = first + p0 * kSmPart * 64;
                todo_last[k] = lay.w;
            }
            if ((item & kSmListHuge) && i % G == blockIdx.x) todo_first[atomicAdd(&n_todo, 1)] = -1 - (int64_t)c;
        }
        __syncthreads();
        const int n = n_todo;
        for (int q = 0; q < n; ++q) {
            if (todo_first[q] < 0) {
                softmax_merge_chunk(row_ptr, out, g_softmax_rec, g_softmax_rows, -1 - todo_first[q]);
                continue;
            }
            const int64_t last = todo_last[q];
            for (int64_t p = todo_first[q]; p <= last; p += G * kSmPart * 64)
                for (int64_t w0 = p + 64 * wave; w0 <= min(last, p + kSmPart * 64 - 1); w0 += kSmBlock)
                    softmax_row_batch(row_ptr, x, out, w0, last, lane);
        }
    }
    for (int64_t i = blockIdx.x; i < n_huge; i += G)
        softmax_merge_chunk(row_ptr, out, g_softmax_rec, g_softmax_rows, g_softmax_list[n_chunks + 1 - i] & kSmListChunk);
}

// SpMM Y[r, :] = sum_p x[p] * H[col_p, :] over a CSR pattern.  Every wave owns kChunk consecutive
// nonzeros; it finds the rows they belong to (search of row_ptr, then a walk) and works through
// them piece by piece.  G lanes span a row of H in float4 (KPL per lane), so 64/G nonzeros of a
// piece are in flight at a time; their partial rows are added across the groups at the end of
// the piece.  A piece that is a whole row is stored; a row cut by a chunk boundary is completed
// with atomic adds into the zeroed Y (the only place where the order of additions can vary from
// run to run).
constexpr int kChunk = 256;

template <int G, int KPL>
__global__ __launch_bounds__(256)
void sddmm_spmm_kernel(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_ind, const float *__restrict__ x,
                       const float *__restrict__ H, float *Y, int64_t n_rows, int64_t nnz, int K)
{
    constexpr int NG = 64 / G;
    const int lane = threadIdx.x & 63, l = lane & (G - 1), g = lane / G;
    const int K4 = K >> 2;
    const int64_t wave = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
    const int64_t p0 = wave * kChunk, p1 = min(nnz, p0 + kChunk);
    if (p0 >= nnz) return;
    // first row whose end lies beyond p0
    int64_t lo = 0, hi = n_rows;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (row_ptr[mid + 1] <= p0) lo = mid + 1; else hi = mid;
    }
    const float4 *H4 = reinterpret_cast<const float4 *>(H);
    for (int64_t r = lo; r < n_rows; ++r) {
        const int64_t rb = row_ptr[r], re = row_ptr[r + 1];
        if (rb >= p1) break;
        const int64_t b = max(rb, p0), e = min(re, p1);
        if (e <= b) continue;
        float4 acc[KPL];
#pragma unroll
        for (int j = 0; j < KPL; ++j) acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int64_t q = b; q < e; q += 64) {
            // 64 entries of the piece at a time into registers, handed to the groups by lane reads
            const int64_t mine = q + lane;
            const int cv = mine < e ? col_ind[mine] : 0;
            const float xv = mine < e ? x[mine] : 0.f;
            const int cnt = (int)min<int64_t>(64, e - q);
            for (int i0 = 0; i0 < cnt; i0 += NG) {  // (a uniform loop: the lane reads below need every lane awake)
                const int i = i0 + g;
                const int c = __shfl(cv, i);
                const float xs = __shfl(xv, i);
                const float4 *hr = H4 + (int64_t)c * K4;
#pragma unroll
                for (int j = 0; j < KPL; ++j) {
                    const int slot = l + j * G;
                    if (slot < K4 && i < cnt) {
                        const float4 h = hr[slot];
                        acc[j].x = fmaf(xs, h.x, acc[j].x); acc[j].y = fmaf(xs, h.y, acc[j].y);
                        acc[j].z = fmaf(xs, h.z, acc[j].z); acc[j].w = fmaf(xs, h.w, acc[j].w);
                    }
                }
            }
        }
        // add the groups' partial rows (lanes with equal l)
#pragma unroll
        for (int off = G; off < 64; off <<= 1) {
#pragma unroll
            for (int j = 0; j < KPL; ++j) {
                acc[j].x += __shfl_xor(acc[j].x, off); acc[j].y += __shfl_xor(acc[j].y, off);
                acc[j].z += __shfl_xor(acc[j].z, off); acc[j].w += __shfl_xor(acc[j].w, off);
            }
        }
        if (g == 0) {
            float *y = Y + r * (int64_t)K;
            const bool whole = (b == rb && e == re);
#pragma unroll
            for (int j = 0; j < KPL; ++j) {
                const int slot = l + j * G;
                if (slot < K4) {
                    if (whole) {
                        *reinterpret_cast<float4 *>(y + 4 * slot) = acc[j];
                    } else {
                        atomicAdd(y + 4 * slot + 0, acc[j].x); atomicAdd(y + 4 * slot + 1, acc[j].y);
                        atomicAdd(y + 4 * slot + 2, acc[j].z); atomicAdd(y + 4 * slot + 3, acc[j].w);
                    }
                }
            }
        }
    }
}

// any K (no alignment assumed): one lane per output column, 64 columns per pass
__global__ __launch_bounds__(256)
void sddmm_spmm_generic_kernel(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_ind, const float *__restrict__ x,
                               const float *__restrict__ H, float *Y, int64_t n_rows, int K)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
    const int64_t n_waves = ((int64_t)gridDim.x * 256) >> 6;
    for (int64_t r = wave; r < n_rows; r += n_waves) {
        const int64_t b = row_ptr[r], e = row_ptr[r + 1];
        for (int k0 = 0; k0 < K; k0 += 64) {
            const int k = k0 + lane;
            float acc = 0.f;
            if (k < K)
                for (int64_t p = b; p < e; ++p) acc = fmaf(x[p], H[(int64_t)col_ind[p] * K + k], acc);
            if (k < K) Y[r * (int64_t)K + k] = acc;
        }
    }
}

__global__ __launch_bounds__(256)
void sddmm_zero_kernel(float4 *dst, int64_t n4)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) dst[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

int last_error(const char *who)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SDDMM_ERR_HIP, "%s: %s", who, hipGetErrorString(e));
    return SDDMM_OK;
}

}  // namespace

namespace sddmm {

// device addresses of the file-scope record arrays on the current device (looked up once per device)
static int softmax_store(float2 **rec, int4 **rows, int32_t **list)
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static float2 *rec_of[kMaxDevices] = {};
    static int4 *rows_of[kMaxDevices] = {};
    static int32_t *list_of[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(SDDMM_ERR_HIP, "sddmm_row_softmax: no usable current device");
    std::lock_guard<std::mutex> lock(mu);
    if (!rec_of[dev]) {
        void *a = nullptr, *b = nullptr, *c = nullptr;
        if ((e = hipGetSymbolAddress(&a, HIP_SYMBOL(g_softmax_rec_store))) != hipSuccess ||
            (e = hipGetSymbolAddress(&b, HIP_SYMBOL(g_softmax_rows_store))) != hipSuccess ||
            (e = hipGetSymbolAddress(&c, HIP_SYMBOL(g_softmax_list_store))) != hipSuccess || !a || !b || !c)
            return fail(SDDMM_ERR_HIP, "sddmm_row_softmax: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        rec_of[dev] = static_cast<float2 *>(a);
        rows_of[dev] = static_cast<int4 *>(b);
        list_of[dev] = static_cast<int32_t *>(c);
    }
    *rec = rec_of[dev];
    *rows = rows_of[dev];
    *list = list_of[dev];
    return SDDMM_OK;
}

int64_t row_softmax_workspace_bytes(int64_t nnz)
{
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    return (((n_chunks * 36 + 8) + 255) / 256) * 256;  // two float2, one int4 and one list item per chunk, and the two lists' lengths
}

int launch_row_softmax(int64_t n_rows, const int32_t *d_row_ptr, const float *d_x, float *d_out, void *stream, void *d_ws, int64_t nnz)
{
    if (n_rows <= 0) return SDDMM_OK;
    float2 *rec = nullptr;
    int4 *rows = nullptr;
    int32_t *list = nullptr;
    if (d_ws) {  // [2 * n_chunks] records, then [n_chunks] chunk layouts, then the two lists: their lengths and [n_chunks] items
        const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
        rec = static_cast<float2 *>(d_ws);
        rows = reinterpret_cast<int4 *>(rec + 2 * n_chunks);
        list = reinterpret_cast<int32_t *>(rows + n_chunks);
    } else if (int rc = softmax_store(&rec, &rows, &list)) {
        return rc;
    }
    // (the entry count lives on the device: the grids are sized for the machine, the kernels stride over the chunks)
    const unsigned grid = 256 * 4;
    hipLaunchKernelGGL(sddmm_row_softmax_rows_kernel, dim3(256), dim3(256), 0, (hipStream_t)stream, d_row_ptr, n_rows, rows, list);
    hipLaunchKernelGGL(sddmm_row_softmax_main_kernel, dim3(6 * grid), dim3(kSmBlock), 0, (hipStream_t)stream, d_row_ptr, n_rows, d_x, d_out,
                       rec, (const int4 *)rows, list);
    hipLaunchKernelGGL(sddmm_row_softmax_merge_kernel, dim3(2 * grid), dim3(kSmBlock), 0, (hipStream_t)stream, d_row_ptr, n_rows, d_x,
                       d_out, (const float2 *)rec, (const int4 *)rows, (const int32_t *)list);
    return last_error("sddmm_row_softmax");
}

}  // namespace sddmm

extern "C" {

int sddmm_row_softmax(int64_t n_rows, const int32_t *d_row_ptr, const float *d_x, float *d_out, void *stream)
{
    if (n_rows < 0 || (n_rows > 0 && (!d_row_ptr || !d_x || !d_out))) return fail(SDDMM_ERR_ARG, "sddmm_row_softmax: bad arguments");
    if (n_rows >= INT32_MAX) return fail(SDDMM_ERR_RANGE, "sddmm_row_softmax: more than 2^31 - 2 rows");
    return launch_row_softmax(n_rows, d_row_ptr, d_x, d_out, stream, nullptr, 0);
}

int sddmm_spmm_csr(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr, const int32_t *d_col_ind,
                   const float *d_x, int32_t K, const float *d_H, float *d_Y, void *stream)
{
    if (n_rows < 0 || n_cols < 0 || nnz < 0 || K < 1) return fail(SDDMM_ERR_ARG, "sddmm_spmm_csr: bad sizes");
    if (n_rows == 0) return SDDMM_OK;
    if (!d_row_ptr || !d_Y || (nnz > 0 && (!d_col_ind || !d_x || !d_H))) return fail(SDDMM_ERR_ARG, "sddmm_spmm_csr: NULL argument");
    if (nnz >= INT32_MAX || n_rows >= INT32_MAX) return fail(SDDMM_ERR_RANGE, "sddmm_spmm_csr: sizes beyond int32 offsets");
    hipStream_t st = (hipStream_t)stream;
    const bool vec = K % 4 == 0 && K <= 2048 && !((((uintptr_t)d_H) | ((uintptr_t)d_Y)) & 15u);
    if (!vec) {
        const unsigned grid = (unsigned)std::min<int64_t>((n_rows + 3) / 4, 256 * 64);
        hipLaunchKernelGGL(sddmm_spmm_generic_kernel, dim3(grid), dim3(256), 0, st, d_row_ptr, d_col_ind, d_x, d_H, d_Y, n_rows, (int)K);
        return last_error("sddmm_spmm_csr");
    }
    // rows cut by a chunk boundary are completed by atomic adds, empty rows stay zero
    const int64_t n4 = n_rows * (int64_t)K / 4;
    hipLaunchKernelGGL(sddmm_zero_kernel, dim3((unsigned)std::min<int64_t>((n4 + 255) / 256, 256 * 32)), dim3(256), 0, st,
                       (float4 *)d_Y, n4);
    if (nnz > 0) {
        const int64_t n_waves = (nnz + kChunk - 1) / kChunk;
        const unsigned grid = (unsigned)((n_waves + 3) / 4);
        const int K4 = K / 4;
#define SPMM(G, KPL) hipLaunchKernelGGL((sddmm_spmm_kernel<G, KPL>), dim3(grid), dim3(256), 0, st, d_row_ptr, d_col_ind, d_x, d_H, d_Y, n_rows, nnz, (int)K)
        if (K4 <= 4) SPMM(4, 1);
        else if (K4 <= 8) SPMM(8, 1);
        else if (K4 <= 16) SPMM(16, 1);
        else if (K4 <= 32) SPMM(32, 1);
        else if (K4 <= 64) SPMM(64, 1);
        else if (K4 <= 128) SPMM(64, 2);
        else if (K4 <= 256) SPMM(64, 4);
        else SPMM(64, 8);
#undef SPMM
    }
    return last_error("sddmm_spmm_csr");
}

}  // extern "C"
