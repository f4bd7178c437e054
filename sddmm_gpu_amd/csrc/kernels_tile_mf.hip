// Tile kernels with a matrix-core share (rows of 128 elements on groups of 8 lanes, one launch
// for all of K), and the kernel that packs their operands.
#include "kernels_tile_impl.hpp"

namespace {

// One workgroup per block of 32 rows: rows [32 blk, 32 blk + 32) of src (through the row list, if
// any; rows at or beyond n_rows read as zero), K slice [k4_off, k4_off + 32) float4, to
// dst[(blk * 32 + p) * 32 + j] = float4 p of row j.  Reads are whole rows; the 16-byte writes of a
// block fill its 16 KB.
__global__ __launch_bounds__(256)
void sddmm_mf_pack_kernel(const float4 *__restrict__ src, const int32_t *__restrict__ rows, int32_t n_rows, int32_t row_k4,
                    int32_t k4_off, float4 *__restrict__ dst, int32_t n_blocks_first, const float4 *__restrict__ src2,
                    const int32_t *__restrict__ rows2, int32_t n_rows2, float4 *__restrict__ dst2)
{
    // (two jobs in one launch: blocks [0, n_blocks_first) pack src, the rest src2)
    int blk = (int)blockIdx.x;
    if (blk >= n_blocks_first) {
        blk -= n_blocks_first;
        src = src2; rows = rows2; n_rows = n_rows2; dst = dst2;
    }
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int f = it * 256 + (int)threadIdx.x, j = f >> 5, p = f & 31;
        const int slot = blk * 32 + j;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (slot < n_rows) {
            const int r = rows ? rows[slot] : slot;
            v = src[(size_t)r * row_k4 + k4_off + p];
        }
        dst[((size_t)blk * 32 + p) * 32 + j] = v;
    }
}

}  // namespace

namespace sddmm {

TileFn tile_kernel_mf(int vmode, int nw, int nwm)
{
#define SDDMM_MF(vm)                                                                       \
    if (vmode == vm) {                                                                     \
        if (nw == 12 && nwm == 4) return (TileFn)sddmm_tile_kernel<8, 4, vm, 12, false, 0, 4>; \
        if (nw == 8 && nwm == 8) return (TileFn)sddmm_tile_kernel<8, 4, vm, 8, false, 0, 8>;   \
        if (nw == 8 && nwm == 4) return (TileFn)sddmm_tile_kernel<8, 4, vm, 8, false, 0, 4>;   \
    }
    SDDMM_MF(0) SDDMM_MF(1) SDDMM_MF(2) SDDMM_MF(3) SDDMM_MF(4)
#undef SDDMM_MF
    return nullptr;
}

void launch_mf_pack(const TileArgs &a, void *stream)
{
    const int row_k4 = a.K >> 2, k4_off = a.k_off >> 2;
    const int nb_h = a.mf_n_cb, nb_w = a.mf_groups;
    hipLaunchKernelGGL(sddmm_mf_pack_kernel, dim3((unsigned)(nb_h + nb_w)), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const float4 *>(a.H), (const int32_t *)nullptr, a.n_cols, row_k4, k4_off,
                       const_cast<float4 *>(a.mf_hp), nb_h, reinterpret_cast<const float4 *>(a.W), a.mf_rows,
                       a.mf_groups * 32, const_cast<float4 *>(a.mf_wp));
}

}  // namespace sddmm
