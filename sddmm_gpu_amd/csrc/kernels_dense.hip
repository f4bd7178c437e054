// Dense-block kernel of the SDDMM engine for gfx950 (MI355X).
//
// Where S has a dense core (heavy rows x popular columns of a power-law
// matrix), the sampled products of a 128 x 128 block are cheaper as one dense
// fp32 contraction on the matrix cores than as gathered dot products on the
// vector ALU: a block of 128 rows (any rows, given by a list) times 128 columns
// (any columns, given by a list) is computed whole with v_mfma_f32_32x32x2_f32
// (plain fp32 in, fp32 accumulate), left in LDS, and the block's nonzeros pick
// their entries from there, scale them by S.val and store them at their own
// positions of the output.  Structural zeros of the block are computed and
// dropped; the planner only hands over blocks dense enough for that to pay.
//
// One workgroup of 4 waves per block, each wave a 64 x 64 quarter (2 x 2 MFMA
// tiles of 32 x 32, 64 accumulator registers).  K runs in chunks of 32: the
// chunk's 128 x 32 slices of the W rows and of the H rows are gathered from
// global memory into registers while the previous chunk is multiplied, then
// written to LDS (double-buffered, rows padded to 144 bytes so that the
// 16-byte operand reads of 16 lanes fall into 64 different banks).
#include <hip/hip_runtime.h>
#include "kernels.hpp"

using namespace sddmm;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float vec4f __attribute__((ext_vector_type(4)));  // (a plain vector type: stays in registers)

constexpr int kT = kDenseTile;        // 128 rows and 128 columns per block
constexpr int kKC = 32;               // K elements per chunk
constexpr int kRowF = kKC + 4;        // floats per staged row (144 bytes)
constexpr int kStageF = kT * kRowF;   // floats per staged operand slice
constexpr int kCRowF = kT + 8;        // floats per row of the result block in LDS
static_assert(4 * kStageF >= kT * kCRowF, "the result block reuses the staging buffers");

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global
// load and store in flight (its workgroup-scope fence), which would drain the requests this kernel
// keeps in the air across its barriers: the next chunk's operands, the block's nonzero list, the
// stores of the block before.  Global memory is never used for communication inside a workgroup here.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__global__ __launch_bounds__(256, 2)
void sddmm_dense_kernel(const DenseArgs a)
{
    __shared__ __attribute__((aligned(16))) float lds[4 * kStageF];  // A0 B0 A1 B1 | result block
    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wr = wave >> 1, wc = wave & 1;  // this wave's 64 x 64 quarter
    const int m = lane & 31, kh = lane >> 5;
    const uint32_t K4 = (uint32_t)(a.K >> 2);
    const int n_chunks = a.K / kKC;
    const vec4f *__restrict__ W4 = reinterpret_cast<const vec4f *>(a.W);
    const vec4f *__restrict__ H4 = reinterpret_cast<const vec4f *>(a.H);
    // staging: thread t carries float4 q of rows r0, r0 + 32, r0 + 64, r0 + 96 of both operands
    const int q = t & 7, r0 = t >> 3;

    // Workgroup b works on slots b, b + grid, ...; its filled slots come first.
    int slot = blockIdx.x;
    if (slot >= a.n_slots) return;
    int2 range = a.slot_range[slot];
    if (range.y <= range.x) return;

    // float4 index of this thread's piece of each of its rows of W and H at chunk 0
    auto load_ids = [&](int s, uint32_t (&wofs)[4], uint32_t (&hofs)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            wofs[i] = (uint32_t)a.slot_rows[s * kT + r0 + 32 * i] * K4 + (uint32_t)q;
            hofs[i] = (uint32_t)a.slot_cols[s * kT + r0 + 32 * i] * K4 + (uint32_t)q;
        }
    };
    vec4f ga[4], gb[4];
    auto fetch = [&](const uint32_t (&wofs)[4], const uint32_t (&hofs)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) ga[i] = W4[wofs[i]];
#pragma unroll
        for (int i = 0; i < 4; ++i) gb[i] = H4[hofs[i]];
    };
    auto stage = [&](int buf) {
        float *A = lds + buf * 2 * kStageF, *B = A + kStageF;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<vec4f *>(A + (r0 + 32 * i) * kRowF + 4 * q) = ga[i];
            *reinterpret_cast<vec4f *>(B + (r0 + 32 * i) * kRowF + 4 * q) = gb[i];
        }
    };
    // One round of the block's nonzero list: 8 entries per thread, strided by the workgroup.
    constexpr int U = 8;
    struct Round { int p[U]; uint32_t rc[U]; float v[U]; };
    auto load_round = [&](Round &r, int first, int n1) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = min(first + 256 * u, n1 - 1);  // clamped: no load behind a branch
            r.p[u] = a.nz_p[idx];
            r.rc[u] = a.nz_rc[idx];
            r.v[u] = a.nz_val ? a.nz_val[idx] : 1.0f;
        }
    };
    const float *Cb = lds;
    auto store_round = [&](Round &r, int first, int n1) {
        if (!a.nz_val && a.val) {
#pragma unroll
            for (int u = 0; u < U; ++u) r.v[u] = a.val[r.p[u]];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float dot = Cb[(r.rc[u] >> 8) * kCRowF + (r.rc[u] & 255u)];
            if (first + 256 * u < n1) a.out[r.p[u]] = a.residual ? r.v[u] - dot : r.v[u] * dot;
        }
    };

    uint32_t wofs[4], hofs[4];
    load_ids(slot, wofs, hofs);
    fetch(wofs, hofs);
    stage(0);
    lds_barrier();
    for (;;) {
        // what the next block needs is requested while this one is computed: its row and column
        // lists now, the first chunk of its operands during this block's last chunk
        const int nslot = slot + (int)gridDim.x;
        int2 nrange = make_int2(0, 0);
        if (nslot < a.n_slots) nrange = a.slot_range[nslot];
        const bool has_next = nrange.y > nrange.x;
        uint32_t nw[4], nh[4];
        load_ids(has_next ? nslot : slot, nw, nh);
        // the first round of this block's nonzero list is requested before the arithmetic starts
        Round r0d;
        load_round(r0d, range.x + t, range.y);

        floatx16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        int par = 0;
        for (int c = 0; c < n_chunks; ++c) {
            const bool last = c + 1 == n_chunks;
            // the next chunk's loads (the last chunk: the next block's first) are issued before this
            // chunk's arithmetic and waited for after it
            uint32_t sw[4], sh[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                sw[i] = last ? nw[i] : wofs[i] + (uint32_t)((c + 1) * (kKC / 4));
                sh[i] = last ? nh[i] : hofs[i] + (uint32_t)((c + 1) * (kKC / 4));
            }
            fetch(sw, sh);
            __builtin_amdgcn_sched_barrier(0);
            const float *A = lds + par * 2 * kStageF, *B = A + kStageF;
            const float *ap = A + (wr * 64 + m) * kRowF + kh * 4;
            const float *bp = B + (wc * 64 + m) * kRowF + kh * 4;
#pragma unroll
            for (int s = 0; s < kKC / 8; ++s) {
                // lanes 0-31 hold elements 8s .. 8s+3 of their row, lanes 32-63 elements 8s+4 .. 8s+7:
                // instruction e of this step multiplies elements 8s+e and 8s+4+e of both operands
                const vec4f a0 = *reinterpret_cast<const vec4f *>(ap + 8 * s);
                const vec4f a1 = *reinterpret_cast<const vec4f *>(ap + 32 * kRowF + 8 * s);
                const vec4f b0 = *reinterpret_cast<const vec4f *>(bp + 8 * s);
                const vec4f b1 = *reinterpret_cast<const vec4f *>(bp + 32 * kRowF + 8 * s);
                const float av[2][4] = {{a0.x, a0.y, a0.z, a0.w}, {a1.x, a1.y, a1.z, a1.w}};
                const float bv[2][4] = {{b0.x, b0.y, b0.z, b0.w}, {b1.x, b1.y, b1.z, b1.w}};
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int i = 0; i < 2; ++i)
#pragma unroll
                        for (int j = 0; j < 2; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i][e], bv[j][e], acc[i][j], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (!last) {
                stage(par ^ 1);
                par ^= 1;
            }
            lds_barrier();
        }
        // the 128 x 128 block of dot products into LDS (over the staging buffers, which everyone has
        // left): register v of lane (m, kh) of tile (i, j) holds row 8*(v/4) + 4*kh + v%4, column m
        float *Cw = lds;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = wr * 64 + i * 32 + 8 * (v >> 2) + 4 * kh + (v & 3);
                    const int col = wc * 64 + j * 32 + m;
                    Cw[row * kCRowF + col] = acc[i][j][v];
                }
        // The block's nonzeros pick their dot products, in rounds of 8 per thread: the first round is
        // here already, the next three are requested together before it is worked on (four rounds
        // cover a block that is half full; fuller ones take further steps of four rounds).
        {
            const int first = range.x + t, n1 = range.y;
            constexpr int R = 256 * U;
            Round r1d, r2d, r3d;
            load_round(r1d, first + R, n1);
            load_round(r2d, first + 2 * R, n1);
            load_round(r3d, first + 3 * R, n1);
            lds_barrier();
            store_round(r0d, first, n1);
            store_round(r1d, first + R, n1);
            store_round(r2d, first + 2 * R, n1);
            store_round(r3d, first + 3 * R, n1);
            for (int f = first + 4 * R; f < n1 + t; f += 4 * R) {  // (uniform bound: first - t + 4R.. < n1)
                load_round(r0d, f, n1);
                load_round(r1d, f + R, n1);
                load_round(r2d, f + 2 * R, n1);
                load_round(r3d, f + 3 * R, n1);
                store_round(r0d, f, n1);
                store_round(r1d, f + R, n1);
                store_round(r2d, f + 2 * R, n1);
                store_round(r3d, f + 3 * R, n1);
            }
        }
        lds_barrier();  // the next block's staging overwrites the result block
        if (!has_next) break;
        stage(0);  // the next block's first chunk has been in registers since this block's last chunk
        lds_barrier();
        slot = nslot;
        range = nrange;
#pragma unroll
        for (int i = 0; i < 4; ++i) { wofs[i] = nw[i]; hofs[i] = nh[i]; }
    }
}

}  // namespace

namespace sddmm {

DenseFn dense_kernel() { return (DenseFn)sddmm_dense_kernel; }

}  // namespace sddmm
