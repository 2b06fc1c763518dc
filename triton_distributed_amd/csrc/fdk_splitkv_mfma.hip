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

// kv heads per workgroup.  Adjacent kv heads of a token are adjacent in the cache, so a workgroup that
// takes two heads reads 512 contiguous bytes per token; measured on MI355X this is the best trade between
// contiguity and the number of independent workgroups.  One head per workgroup is kept where that alone fills
// the compute units without splitting the KV range (no combine pass then).
int mfma_kv_heads_per_wg(int batch, int hkv, int group, int num_cus) {
    const int head_tiles = (group + 15) / 16;
    if (hkv % 2) return 1;
    const int64_t units2 = (int64_t)batch * (hkv / 2) * head_tiles;
    const int64_t units1 = (int64_t)batch * hkv * head_tiles;
    if (units2 >= num_cus) return 2;
    if (units1 >= num_cus) return 1;
    return 2;
}

int mfma_units_per_seq(int hkv, int group, int kv_heads_per_wg) {
    return (hkv / kv_heads_per_wg) * ((group + 15) / 16);
}

int launch_splitkv_mfma(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    switch (p.head_dim) {
        case 64: return launch_splitkv_mfma_d64(p, q_dtype, kv_dtype, stream);
        case 128: return launch_splitkv_mfma_d128(p, q_dtype, kv_dtype, stream);
        case 256: return launch_splitkv_mfma_d256(p, q_dtype, kv_dtype, stream);
        default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace fdk
