// Split-KV paged GQA decode, matrix-core path: dispatch over the head dimension and the plan helpers.
// The kernel itself is in fdk_splitkv_mfma.h.
#include "fdk_device.h"

namespace fdk {

int launch_splitkv_mfma_d64(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream);
int launch_splitkv_mfma_d128(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream);
int launch_splitkv_mfma_d256(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream);

bool mfma_supported(int q_dtype, int kv_dtype, int /*group*/, int head_dim) {
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return false;
    if (q_dtype != FDK_BF16 && q_dtype != FDK_FP16) return false;
    return kv_dtype == q_dtype || kv_dtype == FDK_FP8_E4M3;
}

int mfma_heads_per_wg(int /*group*/) { return 16; }

// kv heads per workgroup.  Adjacent kv heads of a token are adjacent in the cache, so a workgroup that takes
// several heads reads longer contiguous runs per token.  When the (sequence, head block) units alone fill the
// compute units (single pass, no combine) the largest block of 8, 4, 2 or 1 heads that still gives one unit
// per compute unit is taken: with blocks of 4 or 8 heads the workgroup has eight wavefronts, i.e. the whole
// resident set of a compute unit is ONE workgroup whose wavefronts share the tiles and finish together.  Two
// independent 4-wave workgroups per compute unit do not: the older one is served first and the younger one
// runs on alone at the end (measured on MI355X: 386 us -> 364 us for B128, 8 kv heads, fp8 cache).
// Otherwise (the KV range has to be split) two heads per workgroup are the best trade between contiguity and
// the number of independent workgroups.
int mfma_kv_heads_per_wg(int batch, int hkv, int group, int num_cus) {
    const int head_tiles = (group + 15) / 16;
    for (int nh = 8; nh >= 1; nh >>= 1) {
        if (hkv % nh) continue;
        if ((int64_t)batch * (hkv / nh) * head_tiles >= num_cus) return nh;
    }
    return hkv % 2 ? 1 : 2;
}

int mfma_units_per_seq(int hkv, int group, int kv_heads_per_wg) {
    return (hkv / kv_heads_per_wg) * ((group + 15) / 16);
}

int launch_splitkv_mfma(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    if (p.probe) return launch_splitkv_mfma_probe(p, kv_dtype, stream);
    switch (p.head_dim) {
        case 64: return launch_splitkv_mfma_d64(p, q_dtype, kv_dtype, stream);
        case 128: return launch_splitkv_mfma_d128(p, q_dtype, kv_dtype, stream);
        case 256: return launch_splitkv_mfma_d256(p, q_dtype, kv_dtype, stream);
        default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace fdk
