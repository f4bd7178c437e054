// Tile kernels, part 2: the instantiations for value mode 2 (out = dot (no values)).
// The kernel template is compiled in several translation units side by side, which
// divides the build time of the slowest file.
#include "kernels_tile_impl.hpp"

namespace sddmm {

TileFn tile_kernel_part2(const TileVariant &v, int vmode, bool gather, int slice, int nwaves)
{
#define SDDMM_PICK_SLICE(g, kpl, vm, nw, ga)                                                                 \
    (slice == 3 ? fused_slices_kernel<g, kpl, vm, nw, ga>()                                                 \
     : slice == 2 ? (TileFn)sddmm_tile_kernel<g, kpl, (vm == 4 ? 3 : vm), nw, ga, 2>                        \
     : slice == 1 ? (TileFn)sddmm_tile_kernel<g, kpl, vm, nw, ga, 1>                                        \
                  : (TileFn)sddmm_tile_kernel<g, kpl, vm, nw, ga, 0>)
#define SDDMM_PICK(g, kpl, vm)                                                                              \
    (gather ? SDDMM_PICK_SLICE(g, kpl, vm, 4, true)                                                         \
            : (nwaves == 12 ? SDDMM_PICK_SLICE(g, kpl, vm, 12, false) : SDDMM_PICK_SLICE(g, kpl, vm, 16, false)))
#define SDDMM_CASE(g, kpl)                                                                                  \
    if (v.G == g && v.KPL == kpl)                                                                           \
        return SDDMM_PICK(g, kpl, 2);
    SDDMM_CASE(4, 2) SDDMM_CASE(4, 4) SDDMM_CASE(4, 8) SDDMM_CASE(8, 1) SDDMM_CASE(8, 2) SDDMM_CASE(8, 4) SDDMM_CASE(8, 8)
    SDDMM_CASE(16, 4) SDDMM_CASE(16, 8) SDDMM_CASE(32, 4) SDDMM_CASE(32, 8)
#undef SDDMM_CASE
#undef SDDMM_PICK
#undef SDDMM_PICK_SLICE
    return nullptr;
}

}  // namespace sddmm
