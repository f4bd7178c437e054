// Tile kernel variants: which (lanes per nonzero, float4 per lane) pair serves a rank, and
// the table of instantiations (compiled in kernels_tile_p*.hip from kernels_tile_impl.hpp).
#include "kernels.hpp"

namespace sddmm {

TileVariant pick_tile_variant(int K, int want_g)
{
    if (K % 4) return {0, 0};
    const int K4 = K / 4;
    const int cand[][2] = {{4, 2}, {4, 4}, {4, 8}, {8, 1}, {8, 2}, {8, 4}, {8, 8}, {16, 4}, {16, 8}, {32, 4}, {32, 8}};
    TileVariant best{0, 0};
    for (auto &c : cand) {
        if (c[0] * c[1] != K4) continue;
        if (want_g > 0 ? c[0] == want_g : (best.G == 0 || c[1] == 4)) best = {c[0], c[1]};
    }
    return best;
}

TileFn tile_kernel_part0(const TileVariant &v, int vmode, bool gather, int slice, int nwaves);
TileFn tile_kernel_part1(const TileVariant &v, int vmode, bool gather, int slice, int nwaves);
TileFn tile_kernel_part2(const TileVariant &v, int vmode, bool gather, int slice, int nwaves);
TileFn tile_kernel_part3(const TileVariant &v, int vmode, bool gather, int slice, int nwaves);
TileFn tile_kernel_part4(const TileVariant &v, int vmode, bool gather, int slice, int nwaves);

// vmode: see the kernel template (where S.val comes from, which epilogue)
TileFn tile_kernel(const TileVariant &v, int vmode, bool gather, int slice, int nwaves)
{
    switch (vmode) {
    case 0: return tile_kernel_part0(v, vmode, gather, slice, nwaves);
    case 1: return tile_kernel_part1(v, vmode, gather, slice, nwaves);
    case 2: return tile_kernel_part2(v, vmode, gather, slice, nwaves);
    case 3: return tile_kernel_part3(v, vmode, gather, slice, nwaves);
    case 4: return tile_kernel_part4(v, vmode, gather, slice, nwaves);
    }
    return nullptr;
}

}  // namespace sddmm
