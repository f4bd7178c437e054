#pragma once
// Tile kernel of the SDDMM engine for gfx950 (MI355X): column tiles of H in
// LDS, nonzeros streamed in tile order with every (row, tile) run padded to a
// multiple of G positions.
//
// The stream lists S tile by tile (tiles of tile_x columns), rows ascending
// inside a tile; scol holds, instead of the column, the byte offset of the
// column's H row inside the LDS tile.  Each run of one row inside one tile is
// padded to a multiple of G positions (the padding repeats the run's last
// nonzero), so a group of G lanes always works on ONE row: there is no
// per-nonzero row test in the inner loop.  A batch is 64 consecutive stream
// positions, one per lane.  While batch b is computed, the index data of batch
// b+2 (output position, LDS offset, value, W row) and the W row slices of
// batch b+1 are in flight, and the result of batch b-1 is being stored.  Lane l
// of a group holds slice l of the row's W elements; in step I it reads the same
// slice of the H row of one of the group's nonzeros from LDS (in 16-byte pieces;
// the groups sharing one 16-lane LDS phase visit the pieces in different orders,
// so their reads fall into different banks) and accumulates the partial dot
// product in register I.  A halving exchange over the G lanes then leaves the
// whole dot product of nonzero l in lane l, which scales it by S.val and stores
// it at the nonzero's own position in the output.
//
// Short batches (groups of 8 lanes, rows of 128 or 256 elements): the planner
// collects run ends of at most 4 nonzeros, eight to a batch, and writes each of
// them twice into its group's 8 positions.  The two halves of the group then
// work on the same nonzeros, each lane on its own slice, and after 4 of the 8
// steps one more exchange between the halves completes the dot products.
#include <hip/hip_runtime.h>
#include <utility>
#include "kernels.hpp"

using namespace sddmm;

namespace {

// Stream data (positions, LDS offsets, values, W row numbers) is read once per launch: with the
// non-temporal hint it does not displace the W rows and output lines that the caches are needed
// for.  Same-box A/B: the LDS-tile form covering K = 128 in one launch, recommender shape: tile
// kernel 0.638 -> 0.617 ms; the compact stream of K = 32: 0.354 -> 0.384 ms; K slices: no change
// (recommender, K = 256) or + 2 % (banded, K = 512); the gather form + 2 %; on the stores + 12 %
// (the pieces of an output line come from different tiles and have to meet in L2).  So the hint
// is given by the uncompacted single-launch LDS-tile form only.
template <bool STREAMING, class T> __device__ __forceinline__ T ld_meta(const T *p)
{
    if constexpr (STREAMING) return __builtin_nontemporal_load(p);
    else return *p;
}

typedef float vec4f __attribute__((ext_vector_type(4)));  // a plain vector: loadable through an LDS-qualified pointer

__device__ __forceinline__ float dot4(const float4 &a, const float4 &b, float acc)
{
    acc = fmaf(a.x, b.x, acc);
    acc = fmaf(a.y, b.y, acc);
    acc = fmaf(a.z, b.z, acc);
    acc = fmaf(a.w, b.w, acc);
    return acc;
}

// Two ways to walk a group's G nonzeros.
// XORDER (H tile in LDS, rows a multiple of 256 bytes): lane l works, in its step
// I, on the group's nonzero I ^ l, so acc[I] of lane l holds lane l's share of
// nonzero I ^ l.  Every halving step adds to acc[j] the acc[j + S] of the lane S
// away, which belongs to the same nonzero; after the last step acc[0] of lane l is
// the whole dot product of nonzero l.  No lane ever has to choose which of two
// registers to keep and which to send.  (The lanes of a group then read G
// different H rows in one instruction: free in LDS, where only banks count.)
// Otherwise all lanes of a group work on nonzero I in step I and read one
// contiguous piece of its H row (what global memory wants), and each halving
// step selects per lane what to keep and what to send.
// v of lane (lane ^ X).  Distances below 8 are built from DPP lane selects (VALU,
// and the compiler folds them into the add that uses the value): the LDS pipe, which
// a ds_swizzle would occupy, is what the H-tile reads need.
template <int X>
__device__ __forceinline__ int from_lane_xor(int v)
{
    constexpr int kQuadXor1 = 0xB1, kQuadXor2 = 0x4E, kQuadXor3 = 0x1B, kHalfMirror = 0x141;  // dpp_ctrl
    if constexpr (X == 0) return v;
    else if constexpr (X == 1) return __builtin_amdgcn_mov_dpp(v, kQuadXor1, 0xf, 0xf, true);
    else if constexpr (X == 2) return __builtin_amdgcn_mov_dpp(v, kQuadXor2, 0xf, 0xf, true);
    else if constexpr (X == 3) return __builtin_amdgcn_mov_dpp(v, kQuadXor3, 0xf, 0xf, true);
    else if constexpr (X == 7) return __builtin_amdgcn_mov_dpp(v, kHalfMirror, 0xf, 0xf, true);  // lane ^ 7 inside 8 lanes
    else if constexpr (X < 8)  // lane ^ X = (lane ^ 7) ^ (X ^ 7)
        return __builtin_amdgcn_mov_dpp(__builtin_amdgcn_mov_dpp(v, kHalfMirror, 0xf, 0xf, true),
                                        X == 4 ? kQuadXor3 : X == 5 ? kQuadXor2 : kQuadXor1, 0xf, 0xf, true);
    else return __builtin_amdgcn_ds_swizzle(v, (X << 10) | 0x1f);
}

template <int G, int I, bool XORDER>
__device__ __forceinline__ int column_of_step(int v)
{
    if constexpr (XORDER) return from_lane_xor<I>(v);
    else return __builtin_amdgcn_ds_swizzle(v, (I << 5) | (0x1f & ~(G - 1)));  // from lane (lane & ~(G-1)) | I
}

// out[I] = (col of the lane this lane serves in step I) + base, for all G steps.
// With the lane-permuted order and G = 8 or 4 each is ONE v_add_u32 with a DPP lane
// select on its first operand (plus one v_mov for the half-mirrored copy that steps
// 4-6 start from).  Written out because the compiler, left alone, keeps the select
// and the add apart.  Plain VALU instructions only; the leading s_nop covers the two
// wait states a DPP read needs after a VALU write of the same register.
template <int G, bool XORDER>
__device__ __forceinline__ void columns_of_steps(int col, int base, int (&out)[G])
{
    if constexpr (XORDER && G == 8) {
        int hm;
        out[0] = col + base;
        asm("s_nop 1\n\t"
            "v_mov_b32_dpp %[hm], %[c] row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r1], %[c], %[b] quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r2], %[c], %[b] quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r3], %[c], %[b] quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r7], %[c], %[b] row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r4], %[hm], %[b] quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r5], %[hm], %[b] quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r6], %[hm], %[b] quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf bound_ctrl:1"
            : [hm] "=&v"(hm), [r1] "=&v"(out[1]), [r2] "=&v"(out[2]), [r3] "=&v"(out[3]), [r4] "=&v"(out[4]),
              [r5] "=&v"(out[5]), [r6] "=&v"(out[6]), [r7] "=&v"(out[7])
            : [c] "v"(col), [b] "v"(base));
    } else if constexpr (XORDER && G == 4) {
        out[0] = col + base;
        asm("s_nop 1\n\t"
            "v_add_u32_dpp %[r1], %[c], %[b] quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r2], %[c], %[b] quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
            "v_add_u32_dpp %[r3], %[c], %[b] quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1"
            : [r1] "=&v"(out[1]), [r2] "=&v"(out[2]), [r3] "=&v"(out[3])
            : [c] "v"(col), [b] "v"(base));
    } else {
        [&]<int... I>(std::integer_sequence<int, I...>) {
            ((void)(out[I] = column_of_step<G, I, XORDER>(col) + base), ...);
        }(std::make_integer_sequence<int, G>{});
    }
}

template <int S>
__device__ __forceinline__ float xor_lane(float v)
{
    return __int_as_float(from_lane_xor<S>(__float_as_int(v)));
}

// XORDER: lane distance 1 first and the largest last, when one register is left:
// distances 1 and 2 are one v_add with a DPP operand, larger ones cost more.
template <int G, bool XORDER, int S = XORDER ? 1 : G / 2>
__device__ __forceinline__ void transpose_reduce_step(float (&acc)[G], int l)
{
    if constexpr (XORDER) {
        if constexpr (S < G) {
#pragma unroll
            for (int j = 0; j < G; j += 2 * S) acc[j] += xor_lane<S>(acc[j + S]);
            transpose_reduce_step<G, XORDER, S * 2>(acc, l);
        }
    } else if constexpr (S >= 1) {
        const bool upper = (l & S) != 0;
#pragma unroll
        for (int j = 0; j < S; ++j) {
            float keep = upper ? acc[j + S] : acc[j];
            float send = upper ? acc[j] : acc[j + S];
            acc[j] = keep + xor_lane<S>(send);
        }
        transpose_reduce_step<G, XORDER, S / 2>(acc, l);
    }
}

// The matrix-core share of a tile launch, run by the last NWM waves of every workgroup while the
// other waves walk the stream (see TileArgs).  A wave keeps the B operand of one column block
// (32 columns x 128 elements of H: 64 registers) and streams the A operands of its die's row
// groups past it: 64 v_mfma_f32_32x32x2_f32 per (group, block) pair, plain fp32 in and out.  The
// results leave the accumulators directly: accumulator register v of lane l is the dot product of
// row 8 (v / 4) + 4 (l / 32) + v % 4 of the group and column l % 32 of the block; where the row's
// mask has that column's bit, it goes to the row's base position plus the number of set bits below
// the column (a row's nonzeros inside 32 consecutive columns are consecutive in the sorted S).
// ri_slot: 512 bytes of LDS of this wave's own.
// AHEAD: A operands requested ahead of the one in use; CHUNK: results stored per round of value
// loads (both sized by the registers a wave has: 128 with 16 waves per workgroup, 170 with 12).
template <int VMODE, int AHEAD, int CHUNK>
__device__ __forceinline__ void matrix_core_waves(const TileArgs &a, int mw, int nmw, int lane, uint2 *ri_slot)
{
    typedef float v16f __attribute__((ext_vector_type(16)));
    typedef unsigned int v2u __attribute__((ext_vector_type(2)));
    constexpr bool RESIDUAL = VMODE >= 3;
    constexpr bool HASVAL = VMODE != 2;
    const int die = blockIdx.x & 7;
    const int G = a.mf_groups >> 3;
    const int wpd = (int)(gridDim.x >> 3) * nmw;            // matrix-core waves per die
    const int w = (int)(blockIdx.x >> 3) * nmw + mw;        // this wave's number among them
    const int64_t P = (int64_t)G * a.mf_n_cb;               // pairs of the die
    int q = __builtin_amdgcn_readfirstlane((int)(P * w / wpd));
    const int q1 = __builtin_amdgcn_readfirstlane((int)(P * (w + 1) / wpd));
    if (q >= q1) return;
    const int g0 = die * G;
    int cb = __builtin_amdgcn_readfirstlane(q / G), gi = q - cb * G;
    // Operands come through buffer loads: (descriptor in scalar registers) + (scalar byte offset of the
    // pair and step) + (16 bytes per lane), so that no lane computes a 64-bit address.
    constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit elements
    const __amdgpu_buffer_rsrc_t rs_h =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float4 *>(a.mf_hp), 0, a.mf_n_cb << 14, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_w =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float4 *>(a.mf_wp), 0, a.mf_groups << 14, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_ri =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint2 *>(a.mf_rowinfo), 0, (a.mf_groups * a.mf_n_cb) << 8, kRsrcFlags);
    const int ri0 = (g0 * a.mf_n_cb) << 8;
    const int l16 = lane << 4, l8 = (lane & 31) << 3;
    const uint32_t lane_bit = 1u << (lane & 31), lane_lt = lane_bit - 1u;
    const int half4 = (lane >> 5) << 2;
    const uint32_t last = (uint32_t)(a.nnz - 1);
    vec4f b[16];
    auto load_b = [&](int c) {
#pragma unroll
        for (int s = 0; s < 16; ++s)
            b[s] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(rs_h, l16, (c << 14) + s * 1024, 0));
    };
    // row masks and base positions of a pair go through this wave's LDS slot; those of the next
    // pair are requested while this one is computed
    v2u rin = __builtin_amdgcn_raw_buffer_load_b64(rs_ri, l8, ri0 + (q << 8), 0);
    load_b(cb);
    ri_slot[lane] = make_uint2(rin.x, rin.y);
    while (true) {
        const int a_off = (g0 + gi) << 14;
        constexpr int kAhead = AHEAD;
        vec4f aw[kAhead];
#pragma unroll
        for (int s = 0; s < kAhead; ++s)
            aw[s] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(rs_w, l16, a_off + s * 1024, 0));
        __builtin_amdgcn_sched_barrier(0);
        v16f acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[s % kAhead].x, b[s].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[s % kAhead].y, b[s].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[s % kAhead].z, b[s].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[s % kAhead].w, b[s].w, acc, 0, 0, 0);
            if (s + kAhead < 16) {
                aw[s % kAhead] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(rs_w, l16, a_off + (s + kAhead) * 1024, 0));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the next pair's masks and positions arrive while this pair's results are stored
        const int qn = min(q + 1, q1 - 1);
        rin = __builtin_amdgcn_raw_buffer_load_b64(rs_ri, l8, ri0 + (qn << 8), 0);
        __builtin_amdgcn_sched_barrier(0);
        // (the slot was written by this wave: LDS operations of one wave complete in order)
        __builtin_amdgcn_wave_barrier();
        constexpr int kChunk = CHUNK;
#pragma unroll
        for (int h = 0; h < 16 / kChunk; ++h) {
            uint32_t idx[kChunk], has[kChunk];
            float sv[kChunk];
#pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const int v = kChunk * h + u;
                const uint2 r = ri_slot[8 * (v >> 2) + (v & 3) + half4];
                idx[u] = (uint32_t)__builtin_popcount(r.x & lane_lt) + r.y;
                has[u] = r.x & lane_bit;
            }
            if constexpr (HASVAL) {
#pragma unroll
                for (int u = 0; u < kChunk; ++u) sv[u] = a.val[min(idx[u], last)];
            }
#pragma unroll
            for (int u = 0; u < kChunk; ++u) {
                const float d = acc[kChunk * h + u];
                float o;
                if constexpr (RESIDUAL) o = sv[u] - d;
                else if constexpr (HASVAL) o = d * sv[u];
                else o = d;
                if (has[u]) a.out[idx[u]] = o;
            }
        }
        __builtin_amdgcn_wave_barrier();  // (the slot is written again only after these reads)
        ri_slot[lane] = make_uint2(rin.x, rin.y);
        if (++q >= q1) break;
        if (++gi == G) {
            gi = 0;
            ++cb;
            load_b(cb);
        }
    }
}

// VMODE: where S.val comes from -- 0: a.sval (stream order), 1: a.val (sorted
// order, read through the position), 2: nowhere (no scaling); 3 and 4: as 0 and 1
// with the residual epilogue, out = val - dot (K slices after the first: out -= dot,
// no value needed).
//
// The loop is software-pipelined by hand and free of branches around loads, so
// that every wait is for exactly the data needed: while batch b is computed,
// the index data of batch b+2 and the W row slice of batch b+1 are in flight.
// GATHER: no LDS tile; scol holds the column and H rows are read from global
// memory (the stream is then one unit in row order, for rows too short to tile).
// SLICE: 0 = the launch covers all of K (results go to out); 1 = first of several K slices (partial
// results go to a.part, in stream order: one coalesced store per batch); 2 = a later slice (adds to the
// partial result read back from a.part, coalesced, and stores to a.part again or, in the last slice,
// a.to_part == 0, to out).  Only the last slice touches out, with one scattered store per position.
// 3 = all a.n_slices K slices inside this one launch, one after the other (small matrices, where a
// launch costs as much as its work): a wave meets the same positions in every slice, so the partial
// results it left in a.part are its own, and a workgroup barrier between the slices is all the
// ordering needed.
// NWM > 0: the workgroup has NWM more waves, which run the matrix-core share of the launch
// (matrix_core_waves) and take no part in staging or in the stream; the NW vector waves then
// synchronise among themselves through a counter in LDS, since a hardware barrier would wait
// for all waves.
template <int G, int KPL, int VMODE, int NW, bool GATHER, int SLICE, int NWM = 0>
__global__ __launch_bounds__((NW + NWM) * 64)
void sddmm_tile_kernel(const TileArgs a)
{
    constexpr bool FUSED = SLICE == 3;
    constexpr bool ACC = SLICE == 2;
    constexpr bool PART = SLICE >= 1;
    extern __shared__ float4 lds_tile[];
    constexpr int K4 = G * KPL;
    constexpr bool RESIDUAL = VMODE >= 3;
    constexpr bool STREAM_VAL = VMODE == 0 || (VMODE == 3 && !ACC);  // values read in stream order
    constexpr bool SORTED_VAL = VMODE == 1 || (VMODE == 4 && !ACC);  // values read through the position
    constexpr bool XORDER = !GATHER && (K4 % 16 == 0);
    constexpr bool COMPACT = !GATHER && K4 <= 16;  // the compact stream format (see TileArgs)
    constexpr bool STREAM_HINT = !GATHER && !COMPACT && SLICE == 0;  // (see ld_meta)
    // The compact stream serves the thin K slices, where a batch is little arithmetic and the kernel moves
    // at the rate of its requests in flight: 16 waves x 2 batches x 448 bytes of index data per compute unit
    // are 14 KB, and at a microsecond of memory latency 256 compute units then fetch 3.6 TB/s -- what the
    // K = 32 launch measured.  Its index data is therefore requested four batches ahead (the arrays' slack
    // of 256 entries covers exactly the four batches past the end).
    constexpr bool DEEP = COMPACT;
    constexpr int ROW_SHIFT = K4 == 16 ? 8 : K4 == 8 ? 7 : 0;  // log2 of an LDS row in bytes (COMPACT only)
    // SHORTS: a batch may be marked "short" in a.btype: each of its groups then holds at most G/2
    // nonzeros in its first G/2 positions and the same ones again in the other G/2.  With the
    // lane-permuted order the upper half of the lanes then works on the same nonzeros as the lower
    // half, each lane on its own slice, and steps G/2 .. G-1 can be left out: after G/2 steps every
    // half group holds half of each dot product, and one more exchange adds the two.
    constexpr bool SHORTS = tile_variant_shorts(G, KPL, GATHER);
    // Groups that share one 16-lane LDS access phase read the 16-byte pieces of
    // their rows in different orders (piece j ^ rot instead of j), so that their
    // reads fall into different banks whenever rows are a multiple of 256 bytes
    // apart.  NB distinct orders need NB base addresses per row; piece j is then
    // at base[j % NB] + j*G*16, a compile-time offset.
    constexpr int PHASE_GROUPS = (16 / G) >= 1 ? (16 / G) : 1;
    constexpr int NB = GATHER ? 1 : (PHASE_GROUPS < KPL ? PHASE_GROUPS : KPL);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: loop bounds stay in SGPRs
    // barrier among the vector waves: every wave adds one to the counter and waits for the sum to
    // reach NW times the number of barriers so far
    uint32_t sync_target = 0;
    uint32_t *sync_ctr = nullptr;
    if constexpr (NWM > 0) {
        char *extra = reinterpret_cast<char *>(lds_tile) + a.tile_bytes;
        sync_ctr = reinterpret_cast<uint32_t *>(extra);
        if (threadIdx.x == 0) *sync_ctr = 0;
        __syncthreads();  // the only hardware barrier: all waves are still here
        if (wave >= NW) {
            if (a.mf_groups > 0)
                matrix_core_waves<VMODE, (NW + NWM > 12 ? 6 : 8), (NW + NWM > 12 ? 4 : 16)>(a, wave - NW, NWM, lane, reinterpret_cast<uint2 *>(extra + 64) + (wave - NW) * 64);
            return;
        }
    }
    auto wg_sync = [&]() {
        if constexpr (NWM == 0) {
            __syncthreads();
        } else {
            sync_target += NW;
            if (lane == 0) __hip_atomic_fetch_add(sync_ctr, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            while (__hip_atomic_load(sync_ctr, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < sync_target)
                __builtin_amdgcn_s_sleep(1);
        }
    };
    const int l = lane & (G - 1);
    const int rot = (lane / G) & (NB - 1);

    int slot[KPL];      // float4 index inside a row of lane's piece j
    int lane_off[NB];   // byte offset of base t relative to the row start
#pragma unroll
    for (int j = 0; j < KPL; ++j) slot[j] = (j ^ rot) * G + l;
#pragma unroll
    for (int t = 0; t < NB; ++t) lane_off[t] = (l + ((t ^ rot) - t) * G) * 16;
    // LDS addresses are kept as 32-bit integers: the address of this lane's first piece of
    // an H row is (the row's offset in the tile) + lane_base0, added as soon as the offset arrives
    using lds_f4_ptr = const __attribute__((address_space(3))) vec4f *;
    const int lds_base = (int)(uint32_t)(uintptr_t)(lds_f4_ptr)reinterpret_cast<const vec4f *>(lds_tile);
    const int lane_base0 = GATHER ? 0 : lds_base + lane_off[0];
    int base_step[NB];  // base t of a row = base 0 + base_step[t]
#pragma unroll
    for (int t = 0; t < NB; ++t) {
        base_step[t] = lane_off[t] - lane_off[0];
        asm("" : "+v"(base_step[t]));  // one register, not an expression to be re-associated with each use
    }

    const int row_k4 = a.K >> 2;

    // This workgroup's share of the stream: either the items b, b + grid, ... of an item
    // list (each inside one tile), or an equal, 64-aligned range of positions walked unit by unit.
    int lo = 0, hi = 0, unit = 0, n_steps;
    if (a.items) {
        n_steps = (a.n_items - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    } else {
        const int64_t total = a.unit_ptr[a.n_units];
        lo = (int)(((total * blockIdx.x / gridDim.x) + 63) & ~(int64_t)63);
        hi = (blockIdx.x + 1 == gridDim.x) ? (int)total
                                           : (int)(((total * (blockIdx.x + 1) / gridDim.x) + 63) & ~(int64_t)63);
        int a0 = 0, a1 = a.n_units;  // first unit whose end lies beyond lo
        while (a0 < a1) {
            const int mid = (a0 + a1) >> 1;
            if (a.unit_ptr[mid + 1] <= lo) a0 = mid + 1; else a1 = mid;
        }
        unit = a0;
        n_steps = 0;
        for (int u = unit; u < a.n_units && a.unit_ptr[u] < hi; ++u) ++n_steps;
    }
    const int n_slices = FUSED ? a.n_slices : 1;
    for (int sl = 0; sl < n_slices; ++sl) {
    const bool first_slice = sl == 0, last_slice = sl + 1 == n_slices;  // (used by the FUSED form only)
    // this pass covers K elements [k_off, k_off + 4*K4) of rows that are row_k4 float4 long
    const int k_off = a.k_off + sl * 4 * K4;
    const float4 *__restrict__ W4 = reinterpret_cast<const float4 *>(a.W) + (k_off >> 2);
    const float4 *__restrict__ H4 = reinterpret_cast<const float4 *>(a.H) + (k_off >> 2);
    if (FUSED && sl > 0) wg_sync();  // everyone is done with the slice before: its tile, and its partial results are stored
    int cur_tile = -1;
    for (int step = 0; step < n_steps; ++step) {
        int begin, end, tile;
        int type_base = 0;                     // index of the item's first batch in a.btype
        // (constant address space: nothing writes the bits while the kernel runs, and only for such
        // memory does the compiler use scalar loads next to the kernel's own stores)
        using const_u32_ptr = const __attribute__((address_space(4))) uint32_t *;
        const_u32_ptr types = nullptr;         // null: no short batches
        if (a.items) {
            const WorkItem wi = a.items[blockIdx.x + step * gridDim.x];
            begin = wi.begin; end = wi.end; tile = wi.tile;
            if (SHORTS) { type_base = wi.batch_base; types = (const_u32_ptr)(uintptr_t)a.btype; }
        } else {
            begin = max(lo, a.unit_ptr[unit + step]); end = min(hi, a.unit_ptr[unit + step + 1]);
            tile = GATHER ? 0 : a.unit_tile[unit + step];
        }
        if (end <= begin) continue;
        if (!GATHER && tile != cur_tile) {
            if (cur_tile >= 0) wg_sync();  // everyone is done with the previous tile
            cur_tile = tile;
            const int tile_base = tile * a.tile_x;
            const int rows = min(a.tile_x, a.n_cols - tile_base);
            const float4 *src = H4 + (size_t)tile_base * row_k4;
            const int n4 = rows * K4;
            // (eight loads in flight per lane: a workgroup with many tiles in its turn -- a wide matrix --
            // spends its time between tiles waiting for these, one memory latency per round)
            constexpr int kStageUnroll = 8, kStride = NW * 64;
            int i = threadIdx.x;
            for (; i + (kStageUnroll - 1) * kStride < n4; i += kStageUnroll * kStride) {
                float4 v[kStageUnroll];
#pragma unroll
                for (int u = 0; u < kStageUnroll; ++u) {
                    const int ii = i + u * kStride, r = ii / K4, q = ii - r * K4;
                    v[u] = src[(size_t)r * row_k4 + q];
                }
#pragma unroll
                for (int u = 0; u < kStageUnroll; ++u) lds_tile[i + u * kStride] = v[u];
            }
            for (; i < n4; i += kStride) {
                const int r = i / K4, q = i - r * K4;
                lds_tile[i] = src[(size_t)r * row_k4 + q];
            }
            wg_sync();
        }
        const int nb = (end - begin + 63) >> 6;
        // (the division runs on the vector unit; the results are uniform and go back to scalar
        // registers, so that the batch counter and the batch type bits are scalar work)
        const int b0 = __builtin_amdgcn_readfirstlane((int)((int64_t)nb * wave / NW));
        const int b1 = __builtin_amdgcn_readfirstlane((int)((int64_t)nb * (wave + 1) / NW));
        if (b0 >= b1) continue;  // (no barrier below this point inside the tile)
        const int bf = min(b1, (end - begin) >> 6);  // [b0, bf): this wave's batches of 64 whole positions

        // index data of one batch; positions past the item are clamped to its last
        // one (and repeat its work), so no load sits behind a branch
        // Index data of one batch.  The arrays are addressed as (uniform base of the
        // item) + (32-bit byte offset of the lane), the form that needs no per-lane
        // 64-bit arithmetic, and no load sits behind a branch.
        struct Meta { uint32_t wrow, p, o; int col; float sv, old; };  // o: byte offset of the position's fp32 slot inside the item
        const uint32_t last = (uint32_t)(end - begin - 1);
        const char *perm_b = reinterpret_cast<const char *>(COMPACT ? a.pbase + begin / G : a.perm + begin);
        const char *scol_b = COMPACT ? reinterpret_cast<const char *>(a.scol16 + begin)
                                     : reinterpret_cast<const char *>(a.scol + begin);
        const char *sval_b = reinterpret_cast<const char *>(a.sval + begin);
        const char *grow_b = reinterpret_cast<const char *>(a.grow + begin / G);
        // Steady state: batches are requested in order, two ahead of the one computed,
        // with running offsets and no clamp (the batch after a wave's last one is
        // requested and dropped; the arrays have readable slack behind the last position).
        uint32_t o4 = ((uint32_t)(b0 << 6) + (uint32_t)lane) << 2;         // perm, scol, sval
        uint32_t og = (((uint32_t)(b0 << 6) + (uint32_t)lane) / G) << 2;   // grow
        auto issue_meta = [&]() -> Meta {
            Meta m;
            if constexpr (COMPACT) {
                const uint32_t g = ld_meta<STREAM_HINT>(reinterpret_cast<const uint32_t *>(grow_b + og));
                m.wrow = g & ~(uint32_t)(G - 1);
                m.p = ld_meta<STREAM_HINT>(reinterpret_cast<const uint32_t *>(perm_b + og)) + min((uint32_t)l, g & (uint32_t)(G - 1));
                m.col = (int)ld_meta<STREAM_HINT>(reinterpret_cast<const uint16_t *>(scol_b + (o4 >> 1))) << ROW_SHIFT;
            } else {
                m.wrow = ld_meta<STREAM_HINT>(reinterpret_cast<const uint32_t *>(grow_b + og));
                m.p = ld_meta<STREAM_HINT>(reinterpret_cast<const uint32_t *>(perm_b + o4));
                m.col = ld_meta<STREAM_HINT>(reinterpret_cast<const int *>(scol_b + o4));
            }
            m.sv = STREAM_VAL ? ld_meta<STREAM_HINT>(reinterpret_cast<const float *>(sval_b + o4)) : 1.0f;
            m.o = o4;
            o4 += 256;
            og += 256 / G;
            return m;
        };
        // an item's last, partial batch: positions past the end are clamped to the last one
        auto issue_meta_tail = [&](int bi) -> Meta {
            const uint32_t t4 = min((uint32_t)(bi << 6) + (uint32_t)lane, last) << 2;
            Meta m;
            const uint32_t tg = (t4 / (4 * G)) << 2;
            if constexpr (COMPACT) {
                const uint32_t g = *reinterpret_cast<const uint32_t *>(grow_b + tg);
                m.wrow = g & ~(uint32_t)(G - 1);
                m.p = *reinterpret_cast<const uint32_t *>(perm_b + tg) + min((t4 >> 2) & (uint32_t)(G - 1), g & (uint32_t)(G - 1));
                m.col = (int)*reinterpret_cast<const uint16_t *>(scol_b + (t4 >> 1)) << ROW_SHIFT;
            } else {
                m.wrow = *reinterpret_cast<const uint32_t *>(grow_b + tg);
                m.p = *reinterpret_cast<const uint32_t *>(perm_b + t4);
                m.col = *reinterpret_cast<const int *>(scol_b + t4);
            }
            m.sv = STREAM_VAL ? *reinterpret_cast<const float *>(sval_b + t4) : 1.0f;
            m.o = t4;
            return m;
        };
        // ACC (K slices after the first): the previous slices' partial result, requested
        // one batch ahead of its use, from the position's own slot of a.part
        char *part_b = reinterpret_cast<char *>(a.part + begin);
        // (FUSED: the slot is read in every slice and ignored in the first: no load behind a branch)
        auto issue_old = [&](Meta &m) {
            if constexpr (FUSED) {
                const float o = *reinterpret_cast<const float *>(part_b + m.o);
                m.old = first_slice ? 0.f : o;
            } else {
                m.old = ACC ? *reinterpret_cast<const float *>(part_b + m.o) : 0.f;
            }
        };
        // wrow: float4 index of the row's first element in W
        auto issue_w = [&](float4 (&w)[KPL], uint32_t wrow) {
            const float4 *wbase[NB];  // piece j is at wbase[j % NB] + a compile-time offset
            wbase[0] = W4 + (wrow + (uint32_t)slot[0]);
#pragma unroll
            for (int t = 1; t < NB; ++t) wbase[t] = wbase[0] + (slot[t] - slot[0]);
#pragma unroll
            for (int j = 0; j < KPL; ++j) w[j] = wbase[j % NB][(j - j % NB) * G];
        };
        float pend_v;  // result of the batch before, not yet stored
        uint32_t pend_p, pend_o;
        const bool to_part = PART && (FUSED ? !last_slice : a.to_part != 0);  // (uniform)
        // (gather form: a position whose index carries bit 31 is padding that worked on
        // another row's column; its result goes to a scratch line instead of the output)
        // (one store whose address is selected, not a branch around two stores: a branch inside the
        // loop body costs the later slices of a sliced launch 8 % -- 736 against 679 us on the recommender)
        auto flush = [&]() {
            float *dst;
            if constexpr (GATHER) dst = (int32_t)pend_p < 0 ? a.sink + (((blockIdx.x & 255) << 6) + lane) : a.out + pend_p;
            else dst = a.out + pend_p;
            // (a padding position has a slot of its own in a.part)
            if constexpr (PART) dst = to_part ? reinterpret_cast<float *>(part_b + pend_o) : dst;
            *dst = pend_v;
        };
        // c[I]: where the H row this lane works on in step I starts (LDS: byte address of
        // this lane's first piece; gather form: float4 index of the row); cn: the same for the next batch, requested here after the last LDS
        // read so that the latency hides behind the reduction
        auto compute = [&]<bool SHORT>(std::bool_constant<SHORT>, const float4 (&w)[KPL], const Meta &m, const int (&c)[G],
                                       int (&cn)[G], int next_col) {
            constexpr int STEPS = SHORT ? G / 2 : G;
            float v = m.sv;
            if (SORTED_VAL) v = a.val[GATHER ? (m.p & 0x7fffffffu) : m.p];
            float acc[STEPS];
            if constexpr (!GATHER) {
                // The H pieces of step I + 1 are requested before the arithmetic of step I, and the scheduler is kept
                // from moving them back next to their use: an LDS read takes longer than the 16 multiply-adds of a
                // step (same-box A/B, ms per step: recommender K = 128 0.835 -> 0.826, K = 256 1.702 -> 1.691,
                // bag-of-words K = 256 0.0316 -> 0.0299; two steps ahead: no further gain).
                vec4f hb[2][KPL];
                auto rd = [&](vec4f (&h)[KPL], int cI) {
                    int base[NB];  // cI is base 0 already
                    base[0] = cI;
#pragma unroll
                    for (int t = 1; t < NB; ++t) base[t] = cI + base_step[t];
#pragma unroll
                    for (int j = 0; j < KPL; ++j) h[j] = *(lds_f4_ptr)(uintptr_t)(uint32_t)(base[j % NB] + j * G * 16);
                };
                rd(hb[0], c[0]);
                [&]<int... I>(std::integer_sequence<int, I...>) {
                    ((void)[&] {
                        if constexpr (I + 1 < STEPS) rd(hb[(I + 1) & 1], c[I + 1]);
                        __builtin_amdgcn_sched_barrier(0);
                        float s = 0.f;
#pragma unroll
                        for (int j = 0; j < KPL; ++j) {
                            const vec4f h = hb[I & 1][j];
                            s = dot4(w[j], make_float4(h.x, h.y, h.z, h.w), s);
                        }
                        acc[I] = s;
                        __builtin_amdgcn_sched_barrier(0);
                    }(), ...);
                }(std::make_integer_sequence<int, STEPS>{});
            } else {
                [&]<int... I>(std::integer_sequence<int, I...>) {
                    ((void)[&] {
                        const float4 *hr = H4 + (uint32_t)c[I];  // scol: float4 index of the H row
                        float4 h[KPL];
#pragma unroll
                        for (int j = 0; j < KPL; ++j) h[j] = hr[slot[j]];
                        float s = 0.f;
#pragma unroll
                        for (int j = 0; j < KPL; ++j) s = dot4(w[j], h[j], s);
                        acc[I] = s;
                    }(), ...);
                }(std::make_integer_sequence<int, STEPS>{});
            }
            columns_of_steps<G, XORDER>(next_col, lane_base0, cn);
            if constexpr (SHORT) {
                transpose_reduce_step<G / 2, XORDER>(acc, l);  // inside each half group
                acc[0] += xor_lane<G / 2>(acc[0]);             // the other half's slices of the same nonzero
            } else {
                transpose_reduce_step<G, XORDER>(acc, l);
            }
            // The store is left to the start of the next batch (flush): issued here it
            // would sit, unfinished, in front of the loads that batch waits for.  In a
            // whole batch it needs no predicate: a padding position repeats a nonzero of
            // its own group and so writes that nonzero's own result a second time.
            if constexpr (RESIDUAL) pend_v = ACC ? m.old - acc[0] : FUSED ? (first_slice ? v : m.old) - acc[0] : v - acc[0];
            else pend_v = (ACC || FUSED) ? fmaf(acc[0], v, m.old) : acc[0] * v;
            pend_p = m.p;
            pend_o = m.o;
        };

        // the type bits of 32 consecutive batches, held in scalar registers
        uint32_t type_word = 0;
        int type_at = -1;
        auto short_batch = [&](int b) -> bool {
            if constexpr (!SHORTS) return false;
            if (!types) return false;
            const int g = type_base + b;
            if ((g >> 5) != type_at) { type_at = g >> 5; type_word = types[type_at]; }
            return (type_word >> (g & 31)) & 1u;
        };
        auto run = [&](int b, const float4 (&w)[KPL], const Meta &m, const int (&c)[G], int (&cn)[G], int next_col) {
            if (short_batch(b)) compute(std::true_type{}, w, m, c, cn, next_col);
            else compute(std::false_type{}, w, m, c, cn, next_col);
        };

        float4 wa[KPL], wb[KPL];
        int ca[G], cb[G];
        if (b0 < bf) {
            Meta m0 = issue_meta();
            Meta m1 = issue_meta();
            // DEEP: the index data is requested four batches ahead instead of two (see DEEP)
            Meta d2, d3;
            if constexpr (DEEP) { d2 = issue_meta(); d3 = issue_meta(); }
            issue_old(m0);
            issue_w(wa, m0.wrow);
            columns_of_steps<G, XORDER>(m0.col, lane_base0, ca);
            Meta m2 = DEEP ? d2 : issue_meta();
            Meta m3 = DEEP ? d3 : Meta{};
            Meta m4 = DEEP ? issue_meta() : Meta{};
            issue_old(m1);
            issue_w(wb, m1.wrow);
            __builtin_amdgcn_sched_barrier(0);  // keep the requests ahead of the arithmetic
            run(b0, wa, m0, ca, cb, m1.col);
            for (int bi = b0 + 1; bi < bf; bi += 2) {
                flush();
                const Meta n0 = issue_meta();  // batch bi + 2 (DEEP: bi + 4)
                if constexpr (!DEEP) m3 = n0;
                issue_old(m2);
                issue_w(wa, m2.wrow);
                __builtin_amdgcn_sched_barrier(0);
                run(bi, wb, m1, cb, ca, m2.col);
                if (bi + 1 >= bf) break;
                flush();
                const Meta n1 = issue_meta();  // batch bi + 3 (DEEP: bi + 5)
                issue_old(m3);
                issue_w(wb, m3.wrow);
                __builtin_amdgcn_sched_barrier(0);
                run(bi + 1, wa, m2, ca, cb, m3.col);
                m1 = m3;
                if constexpr (DEEP) { m2 = m4; m3 = n0; m4 = n1; }
                else m2 = n1;
            }
            flush();
        }
        if (bf < b1) {
            // the item's last, partial batch: lanes past its end work on the last
            // position once more and store nothing
            Meta mt = issue_meta_tail(bf);
            issue_old(mt);
            issue_w(wa, mt.wrow);
            columns_of_steps<G, XORDER>(mt.col, lane_base0, ca);
            compute(std::false_type{}, wa, mt, ca, cb, mt.col);
            if (begin + (bf << 6) + lane < end) flush();
        }
    }
    }
}

// The all-slices-in-one-launch form exists for slices of 128 elements on groups of 8 lanes only (what the
// planner uses for K > 128); null for the other variants.
template <int G, int KPL, int VMODE, int NW, bool GATHER>
TileFn fused_slices_kernel()
{
    if constexpr (G == 8 && KPL == 4) return (TileFn)sddmm_tile_kernel<G, KPL, VMODE, NW, GATHER, 3>;
    else return nullptr;
}

}  // namespace
