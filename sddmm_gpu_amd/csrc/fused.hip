// The two forms that surround an SDDMM in its machine-learning uses, for gfx950 (MI355X):
// the row-wise softmax of the sampled products (attention scores restricted to the pattern
// of S) and the sparse-times-dense product that consumes them, Y = softmax(S .* W H^T) H.
// Both work on the sorted S directly (CSR pointers + one fp32 per nonzero), so they follow a
// plan's sddmm_execute on the same stream without any re-ordering.
#include <hip/hip_runtime.h>
#include "internal.hpp"

using namespace sddmm;

namespace {

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// Row softmax, one wave per row up to kLongRow entries: the row is read once (up to 8 entries per
// lane stay in registers between the passes), longer rows are read three times by a whole workgroup.
constexpr int kSoftmaxBlock = 256;
constexpr int kRegs = 8;                   // entries per lane kept in registers: rows up to 512 entries
constexpr int kLongRow = 64 * kRegs;

__global__ __launch_bounds__(kSoftmaxBlock)
void sddmm_row_softmax_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, const float *x, float *out)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * kSoftmaxBlock + threadIdx.x) >> 6;
    const int64_t n_waves = ((int64_t)gridDim.x * kSoftmaxBlock) >> 6;
    for (int64_t r = wave; r < n_rows; r += n_waves) {
        const int b = row_ptr[r], e = row_ptr[r + 1];
        const int n = e - b;
        if (n <= 0 || n > kLongRow) continue;  // long rows: the other kernel
        float v[kRegs];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < kRegs; ++i) {
            const int p = b + lane + 64 * i;
            v[i] = p < e ? x[p] : -INFINITY;
            mx = fmaxf(mx, v[i]);
        }
        mx = wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < kRegs; ++i) {
            v[i] = expf(v[i] - mx);  // exp(-inf) = 0 for the lanes past the row's end
            sum += v[i];
        }
        sum = wave_sum(sum);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int i = 0; i < kRegs; ++i) {
            const int p = b + lane + 64 * i;
            if (p < e) out[p] = v[i] * inv;
        }
    }
}

// One workgroup per long row (rows listed nowhere: every workgroup scans its share of the rows
// and takes the long ones it finds; there are few).
__global__ __launch_bounds__(kSoftmaxBlock)
void sddmm_row_softmax_long_kernel(const int32_t *__restrict__ row_ptr, int64_t n_rows, const float *x, float *out)
{
    __shared__ float red[kSoftmaxBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int64_t r = blockIdx.x; r < n_rows; r += gridDim.x) {
        const int b = row_ptr[r], e = row_ptr[r + 1];
        if (e - b <= kLongRow) continue;
        float mx = -INFINITY;
        for (int p = b + threadIdx.x; p < e; p += kSoftmaxBlock) mx = fmaxf(mx, x[p]);
        mx = wave_max(mx);
        __syncthreads();
        if (lane == 0) red[wave] = mx;
        __syncthreads();
        mx = red[0];
#pragma unroll
        for (int w = 1; w < kSoftmaxBlock / 64; ++w) mx = fmaxf(mx, red[w]);
        float sum = 0.f;
        for (int p = b + threadIdx.x; p < e; p += kSoftmaxBlock) sum += expf(x[p] - mx);
        sum = wave_sum(sum);
        __syncthreads();
        if (lane == 0) red[wave] = sum;
        __syncthreads();
        sum = 0.f;
#pragma unroll
        for (int w = 0; w < kSoftmaxBlock / 64; ++w) sum += red[w];
        const float inv = 1.0f / sum;
        for (int p = b + threadIdx.x; p < e; p += kSoftmaxBlock) out[p] = expf(x[p] - mx) * inv;
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

int launch_row_softmax(int64_t n_rows, const int32_t *d_row_ptr, const float *d_x, float *d_out, void *stream)
{
    if (n_rows <= 0) return SDDMM_OK;
    const unsigned grid = (unsigned)std::min<int64_t>((n_rows * 64 + kSoftmaxBlock - 1) / kSoftmaxBlock, 256 * 64);
    hipLaunchKernelGGL(sddmm_row_softmax_kernel, dim3(grid), dim3(kSoftmaxBlock), 0, (hipStream_t)stream, d_row_ptr, n_rows, d_x, d_out);
    const unsigned grid_long = (unsigned)std::min<int64_t>(n_rows, 256 * 8);
    hipLaunchKernelGGL(sddmm_row_softmax_long_kernel, dim3(grid_long), dim3(kSoftmaxBlock), 0, (hipStream_t)stream, d_row_ptr, n_rows,
                       d_x, d_out);
    return last_error("sddmm_row_softmax");
}

}  // namespace sddmm

extern "C" {

int sddmm_row_softmax(int64_t n_rows, const int32_t *d_row_ptr, const float *d_x, float *d_out, void *stream)
{
    if (n_rows < 0 || (n_rows > 0 && (!d_row_ptr || !d_x || !d_out))) return fail(SDDMM_ERR_ARG, "sddmm_row_softmax: bad arguments");
    return launch_row_softmax(n_rows, d_row_ptr, d_x, d_out, stream);
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
