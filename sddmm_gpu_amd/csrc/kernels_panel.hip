// Panel kernel of the SDDMM engine for gfx950 (MI355X): row panels of W stay
// in VGPRs while column tiles of H pass through LDS.
//
// A workgroup owns a panel of rows.  Each group of 8 lanes owns S of them
// ("slots"): the group keeps, per slot, its 1/8 share of the W row (KPL
// float4 per lane), a cursor into the row's nonzeros, and the next 8
// (column, value) pairs of the row, one per lane.  The workgroup then sweeps
// the column tiles of H in ascending order: stage tile j in LDS, barrier, and
// every group consumes, slot by slot, the nonzeros of its rows whose columns
// fall in tile j (rows are column-sorted, so these are the next ones at the
// cursor).  For each such nonzero the group reads the H row from LDS in
// contiguous 16-byte pieces, multiplies with the resident W share, and the
// 8 partial sums of up to 8 nonzeros are reduced together by a butterfly that
// leaves nonzero i's dot product in lane i, which scales it by S.val and
// stores it at the nonzero's own position.  W, the column indices, the values
// and the outputs are each touched once; only H tiles are re-read (once per
// panel), from L2.
#include <hip/hip_runtime.h>
#include <climits>
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

// value of lane I of the caller's 8-lane group
template <int I>
__device__ __forceinline__ int bcast8(int v)
{
    return __builtin_amdgcn_ds_swizzle(v, (I << 5) | 0x18);  // src = (lane & 0x18) | I
}

__device__ __forceinline__ float reduce8(float (&acc)[8], int l)
{
#pragma unroll
    for (int s = 4; s >= 1; s >>= 1) {
        const bool upper = (l & s) != 0;
#pragma unroll
        for (int j = 0; j < s; ++j) {
            float keep = upper ? acc[j + s] : acc[j];
            float send = upper ? acc[j] : acc[j + s];
            acc[j] = keep + __shfl_xor(send, s, 8);
        }
    }
    return acc[0];
}

template <int KPL, int S, int NWAVES>
__global__ __launch_bounds__(NWAVES * 64)
void sddmm_panel_kernel(const PanelArgs a)
{
    extern __shared__ float4 lds_tile[];
    constexpr int KS4 = 8 * KPL;  // float4 per row slice held in LDS
    constexpr int ROT_MASK = (KPL >= 2) ? 1 : 0;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l = lane & 7;
    const int gid = lane >> 3;
    const int rot = gid & ROT_MASK;
    const int K4 = a.K >> 2;
    const int koff4 = a.k_off >> 2;

    int slot_idx[KPL];
#pragma unroll
    for (int j = 0; j < KPL; ++j) slot_idx[j] = ((j + rot) % KPL) * 8 + l;

    const float4 *__restrict__ W4 = reinterpret_cast<const float4 *>(a.W);
    const float4 *__restrict__ H4 = reinterpret_cast<const float4 *>(a.H);

    for (int panel = blockIdx.x; panel < a.n_panels; panel += gridDim.x) {
        int cur[S], end[S], qcol[S];
        float qval[S];
        float4 w[S][KPL];
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int r = a.slot_row[(((size_t)panel * S + s) * NWAVES + wave) * 8 + gid];
            cur[s] = 0; end[s] = 0; qcol[s] = INT_MAX; qval[s] = 0.f;
#pragma unroll
            for (int j = 0; j < KPL; ++j) w[s][j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (r >= 0) {
                cur[s] = a.row_ptr[r];
                end[s] = a.row_ptr[r + 1];
                const float4 *wr = W4 + (size_t)r * K4 + koff4;
#pragma unroll
                for (int j = 0; j < KPL; ++j) w[s][j] = wr[slot_idx[j]];
                const int idx = cur[s] + l;
                if (idx < end[s]) {
                    qcol[s] = a.col_ind[idx];
                    qval[s] = a.val ? a.val[idx] : 1.0f;
                }
            }
        }

        const int tile_first = a.panel_tiles[2 * panel], tile_last = a.panel_tiles[2 * panel + 1];
        for (int tile = tile_first; tile <= tile_last; ++tile) {
            const int tile_base = tile * a.tile_x;
            const int tile_end = min(tile_base + a.tile_x, a.n_cols);
            __syncthreads();  // everyone is done reading the previous tile
            {
                const int n4 = (tile_end - tile_base) * KS4;
                const float4 *src = H4 + (size_t)tile_base * K4 + koff4;
                for (int i = threadIdx.x; i < n4; i += NWAVES * 64) {
                    const int r = i / KS4, q = i - r * KS4;
                    lds_tile[i] = src[(size_t)r * K4 + q];
                }
            }
            __syncthreads();

            bool more;
            do {
                more = false;
#pragma unroll
                for (int s = 0; s < S; ++s) {
                    const bool in = qcol[s] < tile_end;  // a prefix of the 8 queued nonzeros
                    const uint64_t bal = __ballot(in);
                    if (bal != 0) {  // wave-uniform
                        float acc[8];
#define SDDMM_PANEL_STEP(I)                                                                      \
                        acc[I] = 0.f;                                                            \
                        if (bal & (0x0101010101010101ull << I)) {                                \
                            const int c_i = bcast8<I>(qcol[s]);                                  \
                            if (c_i < tile_end) {                                                \
                                const float4 *hr = lds_tile + (size_t)(c_i - tile_base) * KS4;   \
                                _Pragma("unroll") for (int j = 0; j < KPL; ++j)                  \
                                    acc[I] = dot4(w[s][j], hr[slot_idx[j]], acc[I]);             \
                            }                                                                    \
                        }
                        SDDMM_PANEL_STEP(0) SDDMM_PANEL_STEP(1) SDDMM_PANEL_STEP(2) SDDMM_PANEL_STEP(3)
                        SDDMM_PANEL_STEP(4) SDDMM_PANEL_STEP(5) SDDMM_PANEL_STEP(6) SDDMM_PANEL_STEP(7)
#undef SDDMM_PANEL_STEP
                        const float sum = reduce8(acc, l);
                        const int cnt = __popcll((bal >> (gid * 8)) & 0xffull);
                        if (in) {
                            const int idx = cur[s] + l;
                            float res = a.residual ? (a.accumulate ? -sum : qval[s] - sum) : sum * qval[s];
                            if (a.accumulate) res += a.out[idx];
                            a.out[idx] = res;
                        }
                        if (cnt > 0) {  // refill the queue from the new cursor
                            cur[s] += cnt;
                            const int idx = cur[s] + l;
                            const bool ok = idx < end[s];
                            qcol[s] = ok ? a.col_ind[idx] : INT_MAX;
                            qval[s] = ok ? (a.val ? a.val[idx] : 1.0f) : 0.f;
                        }
                        more |= (cnt == 8);
                    }
                }
            } while (__any(more));
        }
    }
}

}  // namespace

namespace sddmm {

PanelVariant pick_panel_variant(int k_slice)
{
    // float4 per lane, slots per group, waves per workgroup
    if (k_slice == 128) return {4, 10, 8};
    if (k_slice == 64) return {2, 16, 8};
    if (k_slice == 32) return {1, 16, 8};
    return {0, 0, 0};
}

PanelFn panel_kernel(const PanelVariant &v)
{
    if (v.KPL == 4 && v.S == 10 && v.NWAVES == 8) return (PanelFn)sddmm_panel_kernel<4, 10, 8>;
    if (v.KPL == 2 && v.S == 16 && v.NWAVES == 8) return (PanelFn)sddmm_panel_kernel<2, 16, 8>;
    if (v.KPL == 1 && v.S == 16 && v.NWAVES == 8) return (PanelFn)sddmm_panel_kernel<1, 16, 8>;
    return nullptr;
}

}  // namespace sddmm
