// Instantiation and dispatch of the VALU split kernel for one (q dtype, fp8-or-not) pair.
// Included by the four fdk_splitkv_valu_*.hip translation units so that they compile in parallel.
#pragma once

#include "fdk_splitkv_valu.h"

namespace fdk {
namespace valu {

template <int QDT, bool FP8, int GT, int HS>
int launch_pm(const SplitParams& p_in, const ValuGeometry& geo, int pm, hipStream_t stream) {
    SplitParams p = p_in;
    const dim3 grid((unsigned)((int64_t)p.batch * p.num_splits * p.hg_blocks * p.head_tiles));
    const dim3 block(64 * geo.nwaves);
    p.wavefronts = geo.nwaves;
    p.grid_x = (int32_t)grid.x;
    const size_t lds = (size_t)(2 * geo.nwaves + (geo.nwaves / 2) * kHeadDim) * HS * GT * sizeof(float);
    switch (pm) {
        case PM_TILE:
            hipLaunchKernelGGL((splitkv_valu_kernel<QDT, FP8, GT, HS, PM_TILE>), grid, block, lds, stream, p);
            break;
        case PM_LOAD:
            hipLaunchKernelGGL((splitkv_valu_kernel<QDT, FP8, GT, HS, PM_LOAD>), grid, block, lds, stream, p);
            break;
        case PM_LANE:
            hipLaunchKernelGGL((splitkv_valu_kernel<QDT, FP8, GT, HS, PM_LANE>), grid, block, lds, stream, p);
            break;
        default:
            hipLaunchKernelGGL((splitkv_valu_kernel<QDT, FP8, GT, HS, PM_LANE_DIV>), grid, block, lds, stream, p);
            break;
    }
    return (int)hipGetLastError();
}

template <int QDT, bool FP8, int GT>
int launch_hs(const SplitParams& p, const ValuGeometry& geo, int pm, hipStream_t stream) {
    return launch_pm<QDT, FP8, GT, 1>(p, geo, pm, stream);   // only HS = 1 is instantiated
}

template <int QDT, bool FP8>
int launch_typed(const SplitParams& p_in, const ValuGeometry& geo, hipStream_t stream) {
    SplitParams p = p_in;
    p.head_tiles = geo.head_tiles;
    p.hg_per_wg = geo.hg_per_wg;
    p.hg_blocks = geo.hg_blocks;
    constexpr int NG = Geo<FP8>::NG;
    const int tpl = NG / geo.hs;
    const int tile_tokens = NJ * (geo.nwaves / geo.hg_per_wg) * tpl;
    int pm;
    if (p.page_shift < 0) pm = PM_LANE_DIV;
    else if (p.page_size % tile_tokens == 0 && p.chunk % tile_tokens == 0) pm = PM_TILE;
    else if (p.page_size % tpl == 0) pm = PM_LOAD;
    else pm = PM_LANE;
    switch (geo.gt) {
        case 1: return launch_hs<QDT, FP8, 1>(p, geo, pm, stream);
        case 2: return launch_hs<QDT, FP8, 2>(p, geo, pm, stream);
        case 4: return launch_hs<QDT, FP8, 4>(p, geo, pm, stream);
        default: return launch_hs<QDT, FP8, 8>(p, geo, pm, stream);
    }
}

}  // namespace valu
}  // namespace fdk
