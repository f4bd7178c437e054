// Plan-free SDDMM over a device CSR that allocates no memory: the row-gather kernel
// with its per-batch side array (the row of every 64th nonzero) built on the device
// into a fixed file-scope array instead of into a plan's own allocations.
#include <hip/hip_runtime.h>
#include <mutex>
#include "internal.hpp"
#include "kernels.hpp"

using namespace sddmm;

namespace {

constexpr int64_t kMaxNnz = SDDMM_NOALLOC_MAX_NNZ;
constexpr int64_t kScratchWords = kMaxNnz / 64 + 64;

// One int32 per batch of 64 nonzeros (16 MiB).  Every GPU the library runs on holds its
// own copy until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress; the device address is looked up once per device below.
static __device__ __align__(256) int32_t scratch[kScratchWords];

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
int32_t *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up once per device).
int scratch_address(int32_t **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(SDDMM_ERR_HIP, "sddmm_csr_noalloc: hipGetDevice failed: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(SDDMM_ERR_HIP, "sddmm_csr_noalloc: device index %d not supported", dev);
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(SDDMM_ERR_HIP, "sddmm_csr_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = static_cast<int32_t *>(p);
    }
    *out = g_scratch_ptr[dev];
    return SDDMM_OK;
}

// batch_row[b] = the row that holds nonzero 64*b, for every b < ceil(nnz / 64): each
// non-empty row writes the batches whose first nonzero lies inside it, so every entry is
// written exactly once per call and nothing of an earlier call is read.
__global__ void batch_rows_kernel(const int32_t *__restrict__ row_ptr, int32_t n_rows, int32_t *__restrict__ batch_row)
{
    for (int64_t r = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; r < n_rows; r += (int64_t)gridDim.x * blockDim.x) {
        const int32_t s = row_ptr[r], e = row_ptr[r + 1];
        for (int32_t b = (s + 63) >> 6; ((int64_t)b << 6) < e; ++b) batch_row[b] = (int32_t)r;
    }
}

}  // namespace

extern "C" int sddmm_csr_noalloc(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                                 const int32_t *d_col_ind, const float *d_val, int32_t K, const float *d_W,
                                 const float *d_H, float *d_out, void *stream)
{
    if (n_rows < 0 || n_cols < 0 || nnz < 0 || K < 1) return fail(SDDMM_ERR_ARG, "sddmm_csr_noalloc: negative size or K < 1");
    if (nnz > kMaxNnz)
        return fail(SDDMM_ERR_RANGE, "sddmm_csr_noalloc: nnz = %lld exceeds the fixed scratch array's limit of %lld nonzeros",
                    (long long)nnz, (long long)kMaxNnz);
    if (n_rows >= INT32_MAX || n_cols >= INT32_MAX) return fail(SDDMM_ERR_RANGE, "sddmm_csr_noalloc: sizes beyond int32 offsets");
    if (nnz == 0) return SDDMM_OK;
    if (n_rows == 0 || n_cols == 0) return fail(SDDMM_ERR_ARG, "sddmm_csr_noalloc: %lld nonzeros in an empty matrix", (long long)nnz);
    if (!d_row_ptr || !d_col_ind || !d_W || !d_H || !d_out) return fail(SDDMM_ERR_ARG, "sddmm_csr_noalloc: NULL device pointer");
    if ((((uintptr_t)d_W | (uintptr_t)d_H) & 15u) && K % 4 == 0)
        return fail(SDDMM_ERR_ARG, "sddmm_csr_noalloc: W and H must be 16-byte aligned");
    int32_t *batch_row = nullptr;
    if (int rc = scratch_address(&batch_row)) return rc;

    const Variant var = (K % 4 == 0) ? pick_variant(K, false) : Variant{0, 0, false};
    const KernelFn fn = var.G ? stream_kernel(var, false) : generic_kernel();
    if (!fn) return fail(SDDMM_ERR_ARG, "sddmm_csr_noalloc: no kernel for K = %d", K);

    hipStream_t s = (hipStream_t)stream;
    const int rows_grid = (int)std::min<int64_t>((n_rows + 255) / 256, 8192);
    hipLaunchKernelGGL(batch_rows_kernel, dim3(rows_grid), dim3(256), 0, s, d_row_ptr, (int32_t)n_rows, batch_row);
    // (the second kernel reads what the first writes: it is not issued when the first could not be)
    if (hipError_t e1 = hipGetLastError(); e1 != hipSuccess)
        return fail(SDDMM_ERR_HIP, "sddmm_csr_noalloc: launch failed: %s", hipGetErrorString(e1));

    KArgs a{};
    a.col_ind = d_col_ind; a.val = d_val; a.W = d_W; a.H = d_H; a.out = d_out;
    a.row_ptr = d_row_ptr; a.batch_row = batch_row; a.n_rows = (int32_t)n_rows;
    a.nnz = (int32_t)nnz; a.K = K; a.n_cols = (int32_t)n_cols; a.tile_x = (int32_t)n_cols;
    // nonzeros per workgroup: up to 8 batches of 64 per wave, fewer when that would leave compute units idle
    const int64_t waves_wanted = 2 * 256 * (kRowGatherBlock / 64);
    const int per_wave = (int)std::clamp<int64_t>(nnz / (64 * waves_wanted), 1, kRowGatherBatchesPerWave);
    a.chunk = 64 * per_wave * (kRowGatherBlock / 64);
    a.generic_perm = var.G == 0;
    const int grid = (int)((nnz + a.chunk - 1) / a.chunk);
    hipLaunchKernelGGL(fn, dim3((unsigned)grid), dim3(kRowGatherBlock), 0, s, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SDDMM_ERR_HIP, "sddmm_csr_noalloc: launch failed: %s", hipGetErrorString(e));
    return SDDMM_OK;
}
