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

// Row softmax.  Every row is worked on whole wherever it fits on chip, so that an entry is read once
// and written once, whatever the rows' lengths (a matrix may hold a few rows of a million entries next
// to millions of rows of ten, so the work is cut by entries, not by rows):
//   short rows (up to kSmChunk entries) are grouped into chunks of consecutive whole rows: chunk c
//        starts with the row that holds entry c * kSmChunk and ends before the row that holds entry
//        (c + 1) * kSmChunk, less than 2 * kSmChunk entries in all.  A workgroup takes a chunk into LDS
//        and gives each row to a lane, a group of lanes, a wave or all its waves, by the row's length:
//        maximum, sum of exponentials, normalisation, all inside LDS; the chunk goes back in one pass.
//   long rows (up to kSmLongMax entries) belong to no chunk: one workgroup each holds the row in
//        registers (the recommender shape keeps 56 % of its entries in rows of more than 4096).
//   huge rows (beyond that) are cut at the multiples of kSmChunk: a piece is stored as exp(x - m) with the
//        piece's own maximum m, (m, sum) goes into a record of the chunk, and a last kernel merges the
//        records of each huge row and scales its pieces.
// The first kernel lays the chunks out (one thread per chunk); all kernels read the number of entries
// from row_ptr[n_rows] on the device and walk the chunks with a grid-sized stride.
constexpr int kSmChunk = 4096;
constexpr int kSmBlock = 256;
constexpr int kSmBuf = 2 * kSmChunk + 8;    // entries of a chunk in LDS: < 2 * kSmChunk, plus the float4 padding at both ends
constexpr int kSmRowsMax = 1024 + 128;     // row pointers of a chunk kept in LDS at a time (with the buffers: 39 KB per workgroup)
constexpr int64_t kSmMaxChunks = ((int64_t)1 << 31) / kSmChunk;
constexpr int kSmLongBlock = 256;                        // threads of a workgroup of the long-row kernel
constexpr int kSmLongQ = 16;                             // float4 per thread
constexpr int kSmLongMax = kSmLongQ * 4 * kSmLongBlock - 8;  // (less what a misaligned start costs)

__device__ __forceinline__ int softmax_row_class(int64_t len) { return len <= kSmChunk ? 0 : len <= kSmLongMax ? 1 : 2; }

// (m, sum) of the pieces of huge rows: [2c] the row that began before chunk c, [2c + 1] the row that ends
// after it; and the layout of each chunk: first entry, end, first row, last row.  The kernels take both
// arrays as arguments: a caller's workspace (sddmm_execute_ws), or these file-scope arrays, 8 + 8 MiB per
// device, held until the process ends -- softmax calls without a workspace that overlap in time on one
// device share them and must not (calls on one stream never do).
static __device__ __align__(256) float2 g_softmax_rec_store[2 * kSmMaxChunks];
static __device__ __align__(256) int4 g_softmax_rows_store[kSmMaxChunks];

// First kernel: the layout, one thread per chunk (two binary searches of row_ptr whose loads the other
// threads' searches hide).  With r the row that holds entry c * kSmChunk, chunk c begins at r's first
// entry (r short), after r's last (r long: the long-row kernel owns it; the chunk may come out empty) or
// at entry c * kSmChunk itself (r huge); it ends where chunk c + 1 would begin if that row were short
// (so a long row that starts past the chunk's rows is left out) or at the multiple (huge).
__global__ __launch_bounds__(256)
void sddmm_row_softmax_rows_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, int4 *__restrict__ g_softmax_rows)
{
    const int64_t nnz = row_ptr[n_rows];
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < n_chunks; c += (int64_t)gridDim.x * blockDim.x) {
        const int64_t p0 = c * kSmChunk, p1 = min(nnz - 1, p0 + kSmChunk);  // (p1 = nnz - 1 in the last chunk: not used there)
        // first row whose end lies beyond p0 / p1
        int64_t lo0 = 0, hi0 = n_rows - 1, lo1 = 0, hi1 = n_rows - 1;
        while (lo0 < hi0 || lo1 < hi1) {
            if (lo0 < hi0) { const int64_t mid = (lo0 + hi0) >> 1; if (row_ptr[mid + 1] <= p0) lo0 = mid + 1; else hi0 = mid; }
            if (lo1 < hi1) { const int64_t mid = (lo1 + hi1) >> 1; if (row_ptr[mid + 1] <= p1) lo1 = mid + 1; else hi1 = mid; }
        }
        int4 lay;
        const int64_t b0 = row_ptr[lo0], e0 = row_ptr[lo0 + 1];
        const int k0 = softmax_row_class(e0 - b0);
        lay.x = (int)(k0 == 0 ? b0 : k0 == 1 ? e0 : p0);
        lay.z = (int)(k0 == 1 ? lo0 + 1 : lo0);
        if (p0 + kSmChunk >= nnz) {
            lay.y = (int)nnz;
            lay.w = (int)(n_rows - 1);
        } else {
            const int64_t b1 = row_ptr[lo1], e1 = row_ptr[lo1 + 1];
            const int k1 = softmax_row_class(e1 - b1);
            lay.y = (int)(k1 == 2 ? p1 : b1);
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

// One row's piece buf[b, e) of a chunk: the lanes that work on it take it into registers (R entries
// each, so that the LDS reads are all in flight together and the row is read and written once), maximum,
// exp(x - max), sum; a whole row is normalised, a piece of a huge row is left as exp(x - max) with
// (max, sum) in *rec.  Three forms, by how many lanes work on the row.

// one lane (rows of a few entries: no lane exchanges at all)
__device__ __forceinline__ void softmax_piece_by_lane(float *buf, int b, int e, bool whole, float2 *rec)
{
    constexpr int R = 8;
    float v[R];
#pragma unroll
    for (int k = 0; k < R; ++k) v[k] = b + k < e ? buf[b + k] : -INFINITY;
    float m = v[0];
#pragma unroll
    for (int k = 1; k < R; ++k) m = fmaxf(m, v[k]);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < R; ++k) {
        v[k] = b + k < e ? exp_nonpositive(v[k] - m) : 0.f;
        sum += v[k];
    }
    const float f = whole ? 1.0f / sum : 1.0f;
#pragma unroll
    for (int k = 0; k < R; ++k) if (b + k < e) buf[b + k] = v[k] * f;
    if (!whole) *rec = make_float2(m, sum);
}

// a group of GW lanes, up to GW * R entries (all lanes of the group call this with the same row; the lane
// exchanges stay inside the group)
template <int GW, int R>
__device__ __forceinline__ void softmax_piece_by_group(float *buf, int b, int e, bool whole, float2 *rec)
{
    const int i0 = b + (threadIdx.x & (GW - 1));
    float v[R];
#pragma unroll
    for (int k = 0; k < R; ++k) v[k] = i0 + k * GW < e ? buf[i0 + k * GW] : -INFINITY;
    float m = v[0];
#pragma unroll
    for (int k = 1; k < R; ++k) m = fmaxf(m, v[k]);
    m = group_max<GW>(m);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < R; ++k) {
        v[k] = i0 + k * GW < e ? exp_nonpositive(v[k] - m) : 0.f;
        sum += v[k];
    }
    sum = group_sum<GW>(sum);
    const float f = whole ? 1.0f / sum : 1.0f;
#pragma unroll
    for (int k = 0; k < R; ++k) if (i0 + k * GW < e) buf[i0 + k * GW] = v[k] * f;
    if (!whole && i0 == b) *rec = make_float2(m, sum);
}

// the whole workgroup, up to kSmBlock * R entries (every thread calls this with the same row).
// red: 2 x (waves per workgroup) floats of LDS
template <int R>
__device__ __forceinline__ void softmax_piece_by_workgroup(float *buf, float *red, int b, int e, bool whole, float2 *rec)
{
    constexpr int NW = kSmBlock / 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i0 = b + threadIdx.x;
    float v[R];
#pragma unroll
    for (int k = 0; k < R; ++k) v[k] = i0 + k * kSmBlock < e ? buf[i0 + k * kSmBlock] : -INFINITY;
    float m = v[0];
#pragma unroll
    for (int k = 1; k < R; ++k) m = fmaxf(m, v[k]);
    m = group_max<64>(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < NW; ++w) m = fmaxf(m, red[w]);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < R; ++k) {
        v[k] = i0 + k * kSmBlock < e ? exp_nonpositive(v[k] - m) : 0.f;
        sum += v[k];
    }
    sum = group_sum<64>(sum);
    if (lane == 0) red[NW + wave] = sum;
    __syncthreads();  // (also: everyone has read the maxima, so the next row may overwrite them)
    sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += red[NW + w];
    const float f = whole ? 1.0f / sum : 1.0f;
#pragma unroll
    for (int k = 0; k < R; ++k) if (i0 + k * kSmBlock < e) buf[i0 + k * kSmBlock] = v[k] * f;
    if (!whole && threadIdx.x == 0) *rec = make_float2(m, sum);
    // (the sums are read before the next row's second barrier, which comes after its first: no barrier needed here)
}

// piece lengths up to which a row is worked on by a lane / a group of 16 lanes / a wave; beyond: the workgroup
constexpr int kSmByLane = 8, kSmBy16 = 192, kSmByWave = 1023;
constexpr int kSmList16 = 2 * kSmChunk / (kSmByLane + 1) + 1, kSmList64 = 2 * kSmChunk / (kSmBy16 + 1) + 1,
              kSmListWg = 2 * kSmChunk / (kSmByWave + 1) + 1;

__global__ __launch_bounds__(kSmBlock, 3)  // (three waves per SIMD: 168 registers, a chunk ahead takes 36 of them)
void sddmm_row_softmax_chunk_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, const float *x, float *out,
                                    float2 *g_softmax_rec, const int4 *__restrict__ g_softmax_rows)
{
    __shared__ __align__(16) float buf[kSmBuf];
    __shared__ int32_t rows_lds[kSmRowsMax];
    __shared__ float red[2 * kSmBlock / 64];
    // rows of the chunk that take more than a lane, by class (index of the row inside the round's window)
    __shared__ uint16_t list16[kSmList16], list64[kSmList64], list_wg[kSmListWg];
    __shared__ int n_listed[3];
    constexpr int kPer = (kSmBuf / 4 + kSmBlock - 1) / kSmBlock;  // float4 per thread and chunk, at most
    const int64_t nnz = row_ptr[n_rows];
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    const bool vec_in = (reinterpret_cast<uintptr_t>(x) & 15u) == 0, vec_out = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    // A chunk travels memory -> registers -> LDS as the float4 pieces from the aligned address below its
    // first entry on; the registers are filled one chunk ahead, so the memory latency of chunk c + grid
    // passes while chunk c is worked on.  The layout of a chunk says what to read, so the layouts are
    // fetched two chunks ahead.
    typedef float vec4 __attribute__((ext_vector_type(4)));  // (a plain vector: stays in registers through the conditional loads)
    vec4 ahead[kPer];
    auto layout_of = [&](int64_t c) { return c < n_chunks ? g_softmax_rows[c] : make_int4(0, 0, 0, 0); };
    auto request = [&](int4 lay) __attribute__((always_inline)) {
        if (vec_in && lay.x < lay.y) {
            const int64_t a0 = lay.x & ~3;
            const int nq = (int)((lay.y - a0 + 3) >> 2);
            const vec4 *src = reinterpret_cast<const vec4 *>(x + a0);
#pragma unroll
            for (int u = 0; u < kPer; ++u) {
                const int q = threadIdx.x + u * kSmBlock;
                // (the last float4 of the array may reach beyond its end: that one is read entry by entry below)
                if (q < nq && a0 + 4 * (int64_t)q + 3 < nnz) ahead[u] = src[q];
            }
        }
    };
    int4 lay_cur = layout_of(blockIdx.x), lay_nxt = layout_of((int64_t)blockIdx.x + gridDim.x);
    request(lay_cur);
    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        const int4 lay_after = layout_of(c + 2 * (int64_t)gridDim.x);
        const int4 lay = lay_cur;
        lay_cur = lay_nxt;
        lay_nxt = lay_after;
        if (lay.x >= lay.y) {  // no short or huge rows here
            request(lay_cur);
            continue;
        }
        const int64_t c0 = lay.x, c1 = lay.y;
        const int64_t a0 = vec_in ? (c0 & ~(int64_t)3) : c0;  // buf[i] holds entry a0 + i
        const int n = (int)(c1 - a0);
        __syncthreads();  // the chunk before has left the buffers
        if (vec_in) {
            const int nq = (n + 3) >> 2;
#pragma unroll
            for (int u = 0; u < kPer; ++u) {
                const int q = threadIdx.x + u * kSmBlock;
                if (q < nq) {
                    if (a0 + 4 * (int64_t)q + 3 < nnz) {
                        reinterpret_cast<vec4 *>(buf)[q] = ahead[u];
                    } else {
                        for (int j = 0; j < 4; ++j) buf[4 * q + j] = a0 + 4 * q + j < nnz ? x[a0 + 4 * q + j] : 0.f;
                    }
                }
            }
        } else {
            for (int i0 = threadIdx.x; i0 < n; i0 += 8 * kSmBlock) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = i0 + u * kSmBlock < n ? x[a0 + i0 + u * kSmBlock] : 0.f;
#pragma unroll
                for (int u = 0; u < 8; ++u) if (i0 + u * kSmBlock < n) buf[i0 + u * kSmBlock] = v[u];
            }
        }
        const int64_t r0 = lay.z, r1 = lay.w;
        // The chunk's row pointers go into LDS, kSmRowsMax - 1 rows at a time (one round unless the chunk is
        // full of empty rows).  These loads are issued before the next chunk is requested, so that waiting
        // for them does not wait for it.
        for (int64_t w0 = r0; w0 <= r1; w0 += kSmRowsMax - 1) {
            const int n_w = (int)(min(r1, w0 + kSmRowsMax - 2) - w0 + 1);  // rows of this round
            if (w0 != r0) __syncthreads();  // the round before has left rows_lds and the lists
            for (int i = threadIdx.x; i <= n_w; i += kSmBlock) rows_lds[i] = row_ptr[w0 + i];
            if (threadIdx.x < 3) n_listed[threadIdx.x] = 0;
            if (w0 == r0) request(lay_cur);
            __syncthreads();
            // (positions inside buf; only a huge row can reach beyond the chunk)
            auto piece = [&](int k, int *b, int *e, bool *whole, float2 **rec) {
                const int64_t rb = rows_lds[k], re = rows_lds[k + 1];
                *b = (int)(max(rb, c0) - a0); *e = (int)(min(re, c1) - a0);
                if (softmax_row_class(re - rb) == 1) *e = *b;  // (no long row lies inside a chunk; should one, it is left alone)
                *whole = rb >= c0 && re <= c1;
                *rec = &g_softmax_rec[2 * c + (rb < c0 ? 0 : 1)];
            };
            // every thread looks at the rows k = t, t + 256, ...: the short ones it does itself, the others it lists
            for (int k = threadIdx.x; k < n_w; k += kSmBlock) {
                int b, e; bool whole; float2 *rec;
                piece(k, &b, &e, &whole, &rec);
                const int len = e - b;
                if (len <= 0) continue;
                if (len <= kSmByLane) softmax_piece_by_lane(buf, b, e, whole, rec);
                else if (len <= kSmBy16) list16[atomicAdd(&n_listed[0], 1)] = (uint16_t)k;
                else if (len <= kSmByWave) list64[atomicAdd(&n_listed[1], 1)] = (uint16_t)k;
                else list_wg[atomicAdd(&n_listed[2], 1)] = (uint16_t)k;
            }
            __syncthreads();
            const int n16 = n_listed[0], n64 = n_listed[1], n_wg = n_listed[2];
            for (int q = 0; q < n_wg; ++q) {
                int b, e; bool whole; float2 *rec;
                piece(list_wg[q], &b, &e, &whole, &rec);
                if (e - b <= 8 * kSmBlock) softmax_piece_by_workgroup<8>(buf, red, b, e, whole, rec);
                else softmax_piece_by_workgroup<kSmChunk / kSmBlock>(buf, red, b, e, whole, rec);
            }
            for (int q = threadIdx.x >> 6; q < n64; q += kSmBlock / 64) {
                int b, e; bool whole; float2 *rec;
                piece(list64[q], &b, &e, &whole, &rec);
                if (e - b <= 6 * 64) softmax_piece_by_group<64, 6>(buf, b, e, whole, rec);
                else softmax_piece_by_group<64, (kSmByWave + 63) / 64>(buf, b, e, whole, rec);
            }
            for (int q = threadIdx.x >> 4; q < n16; q += kSmBlock / 16) {
                int b, e; bool whole; float2 *rec;
                piece(list16[q], &b, &e, &whole, &rec);
                if (e - b <= 4 * 16) softmax_piece_by_group<16, 4>(buf, b, e, whole, rec);
                else softmax_piece_by_group<16, kSmBy16 / 16>(buf, b, e, whole, rec);
            }
        }
        __syncthreads();
        const int lo = (int)(c0 - a0);  // 0 .. 3: the entries before belong to the chunk or the long row before
        if (vec_in && vec_out) {
            float4 *dst = reinterpret_cast<float4 *>(out + a0);
            const int nq = (n + 3) >> 2;
#pragma unroll
            for (int u = 0; u < kPer; ++u) {
                const int q = threadIdx.x + u * kSmBlock, i = 4 * q;
                if (q >= nq) continue;
                if (i >= lo && i + 4 <= n) {
                    dst[q] = reinterpret_cast<const float4 *>(buf)[q];
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) if (i + j >= lo && i + j < n) out[a0 + i + j] = buf[i + j];
                }
            }
        } else {
            for (int i = lo + threadIdx.x; i < n; i += kSmBlock) out[a0 + i] = buf[i];
        }
    }
}

// One long row [rb, re) by a workgroup of kSmLongBlock threads, the row held in registers (4 * NQ floats
// per thread): read once, written once.  x 16-byte aligned: float4 pieces counted from the aligned
// address below the row's start (entries outside the row are masked); otherwise single entries, strided.
template <int NQ>
__device__ __forceinline__ void softmax_long_row(const float *x, float *out, int64_t rb, int64_t re, int64_t nnz, bool vec_in,
                                                 bool vec_out, float *red)
{
    constexpr int NW = kSmLongBlock / 64;
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
            const int p = 4 * (t + k * kSmLongBlock);
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
            const int p = t + k * kSmLongBlock;
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
    const float inv = 1.0f / sum;
    if (vec_in) {
#pragma unroll
        for (int k = 0; k < NQ; ++k) {
            const int p = 4 * (t + k * kSmLongBlock);
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
            const int p = t + k * kSmLongBlock;
            if (p < end) outr[p] = f[k] * inv;
        }
    }
    // (the next row writes its maxima after this row's second barrier and its sums after its own first: no barrier needed here)
}

// The long rows.  A long row holds the multiple of kSmChunk that follows its first entry, so it is the
// row after the last row of the chunk whose window [c * kSmChunk, (c + 1) * kSmChunk) it starts in.
// Workgroup b looks at the chunks b, b + grid, ...: first at many of them at once, a thread per chunk
// (three dependent loads each, which a walk chunk by chunk would pay for one after the other), the long
// rows that start in them collected in a list; then the list row by row.
__global__ __launch_bounds__(kSmLongBlock, 4)  // (four waves per SIMD = 128 registers: four rows in flight per compute unit)
void sddmm_row_softmax_long_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, const float *x, float *out,
                                   const int4 *__restrict__ g_softmax_rows)
{
    __shared__ float red[2 * kSmLongBlock / 64];
    __shared__ int2 todo[kSmLongBlock];
    __shared__ int n_todo;
    const int64_t nnz = row_ptr[n_rows];
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    const bool vec_in = (reinterpret_cast<uintptr_t>(x) & 15u) == 0, vec_out = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    for (int64_t base = blockIdx.x; base < n_chunks; base += (int64_t)gridDim.x * kSmLongBlock) {
        __syncthreads();  // the list of the round before has been worked off
        if (threadIdx.x == 0) n_todo = 0;
        __syncthreads();
        const int64_t c = base + (int64_t)threadIdx.x * gridDim.x;
        if (c < n_chunks) {
            const int64_t r = (int64_t)g_softmax_rows[c].w + 1;
            if (r < n_rows) {
                const int64_t rb = row_ptr[r], re = row_ptr[r + 1];
                if (rb >= c * kSmChunk && rb < (c + 1) * kSmChunk && softmax_row_class(re - rb) == 1)
                    todo[atomicAdd(&n_todo, 1)] = make_int2((int)rb, (int)re);
            }
        }
        __syncthreads();
        const int n = n_todo;
        for (int q = 0; q < n; ++q) {
            const int64_t rb = todo[q].x, re = todo[q].y;
            if (re - rb <= 8 * 4 * kSmLongBlock - 8) softmax_long_row<8>(x, out, rb, re, nnz, vec_in, vec_out, red);
            else softmax_long_row<kSmLongQ>(x, out, rb, re, nnz, vec_in, vec_out, red);
        }
    }
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

// Last kernel: the pieces of huge rows are scaled to the whole row's maximum and sum.  A chunk holds at
// most two of them: at its beginning (the row came from the chunk before, or fills this one and goes on)
// and at its end.
__global__ __launch_bounds__(kSmBlock)
void sddmm_row_softmax_merge_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, float *out,
                                    const float2 *__restrict__ g_softmax_rec, const int4 *__restrict__ g_softmax_rows)
{
    const int64_t nnz = row_ptr[n_rows];
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    // (like the long-row kernel: the chunks are looked at many at a time, the few with work listed)
    __shared__ int todo[kSmBlock];
    __shared__ int n_todo;
    for (int64_t base = blockIdx.x; base < n_chunks; base += (int64_t)gridDim.x * kSmBlock) {
        __syncthreads();
        if (threadIdx.x == 0) n_todo = 0;
        __syncthreads();
        {
            const int64_t c = base + (int64_t)threadIdx.x * gridDim.x;
            if (c < n_chunks) {
                const int4 lay = g_softmax_rows[c];
                if (lay.x < lay.y) {
                    const int64_t r0 = lay.z, r1 = lay.w;
                    if (softmax_row_class((int64_t)row_ptr[r0 + 1] - row_ptr[r0]) == 2 ||
                        softmax_row_class((int64_t)row_ptr[r1 + 1] - row_ptr[r1]) == 2)
                        todo[atomicAdd(&n_todo, 1)] = threadIdx.x;
                }
            }
        }
        __syncthreads();
        const int n = n_todo;
        for (int q = 0; q < n; ++q) {
            const int64_t c = base + (int64_t)todo[q] * gridDim.x;
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
    }
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
static int softmax_store(float2 **rec, int4 **rows)
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static float2 *rec_of[kMaxDevices] = {};
    static int4 *rows_of[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(SDDMM_ERR_HIP, "sddmm_row_softmax: no usable current device");
    std::lock_guard<std::mutex> lock(mu);
    if (!rec_of[dev]) {
        void *a = nullptr, *b = nullptr;
        if ((e = hipGetSymbolAddress(&a, HIP_SYMBOL(g_softmax_rec_store))) != hipSuccess ||
            (e = hipGetSymbolAddress(&b, HIP_SYMBOL(g_softmax_rows_store))) != hipSuccess || !a || !b)
            return fail(SDDMM_ERR_HIP, "sddmm_row_softmax: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        rec_of[dev] = static_cast<float2 *>(a);
        rows_of[dev] = static_cast<int4 *>(b);
    }
    *rec = rec_of[dev];
    *rows = rows_of[dev];
    return SDDMM_OK;
}

int64_t row_softmax_workspace_bytes(int64_t nnz)
{
    const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
    return ((n_chunks * 32 + 255) / 256) * 256;  // two float2 and one int4 per chunk
}

int launch_row_softmax(int64_t n_rows, const int32_t *d_row_ptr, const float *d_x, float *d_out, void *stream, void *d_ws, int64_t nnz)
{
    if (n_rows <= 0) return SDDMM_OK;
    float2 *rec = nullptr;
    int4 *rows = nullptr;
    if (d_ws) {  // [2 * n_chunks] records, then [n_chunks] chunk layouts
        const int64_t n_chunks = (nnz + kSmChunk - 1) / kSmChunk;
        rec = static_cast<float2 *>(d_ws);
        rows = reinterpret_cast<int4 *>(rec + 2 * n_chunks);
    } else if (int rc = softmax_store(&rec, &rows)) {
        return rc;
    }
    // (the entry count lives on the device: the grid is sized for the machine, the kernels stride over the chunks)
    const unsigned grid = 256 * 4;
    const unsigned grid_chunk = 256 * 3;  // (168 registers: three workgroups per compute unit)
    hipLaunchKernelGGL(sddmm_row_softmax_rows_kernel, dim3(256), dim3(256), 0, (hipStream_t)stream, d_row_ptr, n_rows, rows);
    hipLaunchKernelGGL(sddmm_row_softmax_chunk_kernel, dim3(grid_chunk), dim3(kSmBlock), 0, (hipStream_t)stream, d_row_ptr, n_rows, d_x, d_out,
                       rec, (const int4 *)rows);
    hipLaunchKernelGGL(sddmm_row_softmax_merge_kernel, dim3(2 * grid), dim3(kSmBlock), 0, (hipStream_t)stream, d_row_ptr, n_rows, d_out,
                       (const float2 *)rec, (const int4 *)rows);
    // (the long rows are touched by neither kernel above: this one could run anywhere after the first)
    hipLaunchKernelGGL(sddmm_row_softmax_long_kernel, dim3(2 * grid), dim3(kSmLongBlock), 0, (hipStream_t)stream, d_row_ptr, n_rows, d_x, d_out,
                       (const int4 *)rows);
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
