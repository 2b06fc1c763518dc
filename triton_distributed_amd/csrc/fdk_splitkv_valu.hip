// VALU split kernel: geometry selection and dtype dispatch (kernels: fdk_splitkv_valu.h).
#include "fdk_splitkv_valu.h"

namespace fdk {

namespace {

int pow2_floor(int x) {
    int r = 1;
    while (r * 2 <= x) r *= 2;
    return r;
}

}  // namespace

int valu_heads_per_wg(int group) {
    if (group <= 1) return 1;
    if (group <= 2) return 2;
    if (group <= 4) return 4;
    return 8;
}

bool valu_supported(int q_dtype, int kv_dtype, int /*group*/, int head_dim) {
    if (head_dim != kHeadDim) return false;
    if (q_dtype != FDK_BF16 && q_dtype != FDK_FP16) return false;
    return kv_dtype == q_dtype || kv_dtype == FDK_FP8_E4M3;
}

namespace valu {

ValuGeometry choose_geometry(const SplitParams& p, int kv_dtype) {
    ValuGeometry g;
    g.gt = valu_heads_per_wg(p.group);
    g.head_tiles = (p.group + g.gt - 1) / g.gt;
    const bool contiguous = p.k_sh == kHeadDim && p.v_sh == kHeadDim;
    // One kv head per wave load (HS = 1).  The kernel template also supports loads that span several adjacent
    // heads; on MI355X that variant measured slower for this issue-bound path (fewer, fatter workgroups).
    g.hs = 1;
    (void)contiguous;
    (void)kv_dtype;
    const int n_hg = p.hkv / g.hs;
    g.nwaves = 4;
    int per = pow2_floor(n_hg < g.nwaves ? n_hg : g.nwaves);
    while (n_hg % per) per >>= 1;
    g.hg_per_wg = per;
    g.hg_blocks = n_hg / per;
    // LDS of the wave merge must stay within 64 KB
    while (g.nwaves > 4 &&
           (size_t)(2 * g.nwaves + (g.nwaves / 2) * kHeadDim) * g.hs * g.gt * sizeof(float) > 64 * 1024)
        g.nwaves >>= 1;
    if (g.hg_per_wg > g.nwaves) {
        g.hg_per_wg = g.nwaves;
        g.hg_blocks = n_hg / g.hg_per_wg;
    }
    return g;
}

}  // namespace valu

int valu_units_per_seq(int hkv, int group, bool heads_contiguous, int kv_dtype) {
    SplitParams p;
    p.group = group;
    p.hkv = hkv;
    p.k_sh = p.v_sh = heads_contiguous ? kHeadDim : 0;
    const valu::ValuGeometry g = valu::choose_geometry(p, kv_dtype);
    return g.hg_blocks * g.head_tiles;
}

int launch_splitkv_valu(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    const valu::ValuGeometry geo = valu::choose_geometry(p, kv_dtype);
    const bool fp8 = kv_dtype == FDK_FP8_E4M3;
    if (q_dtype == FDK_BF16)
        return fp8 ? valu::launch_typed<FDK_BF16, true>(p, geo, stream) : valu::launch_typed<FDK_BF16, false>(p, geo, stream);
    return fp8 ? valu::launch_typed<FDK_FP16, true>(p, geo, stream) : valu::launch_typed<FDK_FP16, false>(p, geo, stream);
}

}  // namespace fdk
