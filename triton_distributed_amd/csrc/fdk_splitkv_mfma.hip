// Split-KV paged GQA decode, matrix-core path: dispatch over the head dimension and the plan helpers.
// The kernel itself is in fdk_splitkv_mfma.h.
#include "fdk_device.h"

namespace fdk {

#define FDK_DECLARE_MFMA(D)                                                                                   \
    int launch_splitkv_mfma_d##D(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream);        \
    int launch_splitkv_mfma_d##D##_queue(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream); \
    int launch_splitkv_mfma_d##D##_bal(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream);
FDK_DECLARE_MFMA(64)
FDK_DECLARE_MFMA(128)
FDK_DECLARE_MFMA(256)
FDK_DECLARE_MFMA(192)            // rows of two segments (128 + 64)
FDK_DECLARE_MFMA(192v128)        // ... with V rows of 128 values
FDK_DECLARE_MFMA(576v512)        // 512 + 64, V rows of 512
FDK_DECLARE_MFMA(576v512_shared) // ... large q-head groups: wavefronts share the staged tiles
FDK_DECLARE_MFMA(128_tiled)      // rows of 128 values, more than 16 q heads per kv head: q-head tiles on one XCD
#undef FDK_DECLARE_MFMA
// (the same rule as mfma_work_mode in the kernel header, which this file does not include)
static int work_mode_of(const SplitParams& p) {
    const int hg_per_wg = (p.hg_per_wg < 1 || p.hkv % p.hg_per_wg) ? 1 : p.hg_per_wg;
    const int tile_heads = p.tile_heads > 16 ? p.tile_heads : 16;       // q heads of a kv head per workgroup
    const int64_t items = (int64_t)p.batch * p.num_splits * (p.hkv / hg_per_wg) * ((p.group + tile_heads - 1) / tile_heads);
    // two 4-wave workgroups fit a compute unit; of the kernels that cover 64 q heads per workgroup, one
    const int resident = (tile_heads > 16 ? 1 : 2) * (p.num_cus > 0 ? p.num_cus : 256);
    return p.balanced ? 2 : (p.counters != nullptr && !p.direct && items > resident) ? 1 : 0;
}

// head_dim (q and K rows) / v_head_dim (V and output rows): 64, 128, 256 with V rows alike, 16-bit and fp8 caches;
// 192 / 192, 192 / 128 and 576 / 512 - rows of two power-of-two segments, as the reference's BLOCK_HEAD_DIM + BLOCK_DPE
// (flash_decode.py:103-109) - 16-bit and fp8 caches (an fp8 cache: the kernels with a tile of 16 q heads per wavefront)
bool mfma_supported(int q_dtype, int kv_dtype, int /*group*/, int head_dim, int v_head_dim) {
    if (q_dtype != FDK_BF16 && q_dtype != FDK_FP16) return false;
    if (head_dim == v_head_dim && (head_dim == 64 || head_dim == 128 || head_dim == 256))
        return kv_dtype == q_dtype || kv_dtype == FDK_FP8_E4M3;
    const bool two_segments = (head_dim == 192 && (v_head_dim == 192 || v_head_dim == 128)) || (head_dim == 576 && v_head_dim == 512);
    return two_segments && (kv_dtype == q_dtype || kv_dtype == FDK_FP8_E4M3);
}

// q heads of one kv head that a workgroup covers: a tile of 16 (a wavefront per kv head), or 64 where the rows are long -
// latent attention, up to 128 q heads on one kv head of 576 + 512 values - and the kernels of fdk_splitkv_mfma_shared.h
// load and stage every tile once for four tiles of 16 q heads.  16-bit caches: whatever the group, the rows of those
// kernels go straight from memory into LDS, which beats the 16-head kernels even where most of a workgroup's wavefronts
// have no q heads and only help to load (batch 32 x 4096 tokens, 8 / 16 / 32 q heads: 51 / 52 / 56 us against 75 / 77 /
// 115 us).  e4m3 caches, whose values have to be converted on the way: from 17 q heads on (8 / 16 / 32 q heads: 52 / 53 /
// 58 us against 50 / 52 / 90 us).
int mfma_heads_per_wg(int group, int row_values, int kv_dtype) {
    return row_values > 512 && (kv_dtype != FDK_FP8_E4M3 || group > 16) ? 64 : 16;
}

// kv heads per workgroup.  Adjacent kv heads of a token are adjacent in the cache, so a workgroup that takes
// several heads reads longer contiguous runs per token.  When the (sequence, head block) units alone fill the
// compute units (single pass, no combine) the largest block of 8, 4, 2 or 1 heads that still gives one unit
// per compute unit is taken: with blocks of 4 or 8 heads the workgroup has eight wavefronts, i.e. the whole
// resident set of a compute unit is ONE workgroup whose wavefronts share the tiles and finish together.  Two
// independent 4-wave workgroups per compute unit do not: the older one is served first and the younger one
// runs on alone at the end (measured on MI355X: 386 us -> 364 us for B128, 8 kv heads, fp8 cache).
// Otherwise (the KV range has to be split) two heads per workgroup are the best trade between contiguity and
// the number of independent workgroups.
// (Rows of more than 512 values per token and kv head, K and V together: at most two heads, i.e. the four wavefronts
// that the registers and the LDS of a compute unit hold at that size.)
int mfma_kv_heads_per_wg(int batch, int hkv, int group, int num_cus, int row_values, int kv_dtype) {
    if (mfma_heads_per_wg(group, row_values, kv_dtype) > 16) return 1;   // the shared-tile kernels: one kv head, 64 q heads
    const int head_tiles = (group + 15) / 16;
    for (int nh = row_values > 512 ? 2 : 8; nh >= 1; nh >>= 1) {
        if (hkv % nh) continue;
        if ((int64_t)batch * (hkv / nh) * head_tiles >= num_cus) return nh;
    }
    return hkv % 2 ? 1 : 2;
}

int mfma_units_per_seq(int hkv, int group, int kv_heads_per_wg, int tile_heads) {
    return (hkv / kv_heads_per_wg) * ((group + tile_heads - 1) / tile_heads);
}

int launch_splitkv_mfma(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    if (p.probe) return launch_splitkv_mfma_probe(p, kv_dtype, stream);
    // the ways of handing out pieces are kernels of their own, instantiated in translation units of their own
    const int mode = work_mode_of(p);
#define FDK_MFMA_CASE(D, KEY)                                                                   \
    case KEY:                                                                                   \
        return mode == 2 ? launch_splitkv_mfma_d##D##_bal(p, q_dtype, kv_dtype, stream)         \
             : mode == 1 ? launch_splitkv_mfma_d##D##_queue(p, q_dtype, kv_dtype, stream)       \
                         : launch_splitkv_mfma_d##D(p, q_dtype, kv_dtype, stream);
    if (p.tile_heads > 16) {
        switch (p.head_dim * 1024 + p.v_head_dim) {
            FDK_MFMA_CASE(576v512_shared, 576 * 1024 + 512)
            default: return (int)hipErrorInvalidValue;
        }
    }
    if (p.v_head_dim != p.head_dim) {
        switch (p.head_dim * 1024 + p.v_head_dim) {
            FDK_MFMA_CASE(192v128, 192 * 1024 + 128)
            FDK_MFMA_CASE(576v512, 576 * 1024 + 512)
            default: return (int)hipErrorInvalidValue;
        }
    }
    // several q-head tiles per kv head read the same rows: the kernels that keep them on one XCD (no single-launch form)
    if (p.head_dim == 128 && p.group > 16 && !p.fused) {
        switch (p.head_dim) { FDK_MFMA_CASE(128_tiled, 128) }
    }
    switch (p.head_dim) {
        FDK_MFMA_CASE(64, 64)
        FDK_MFMA_CASE(128, 128)
        FDK_MFMA_CASE(256, 256)
        FDK_MFMA_CASE(192, 192)
        default: return (int)hipErrorInvalidValue;
    }
#undef FDK_MFMA_CASE
}

}  // namespace fdk
