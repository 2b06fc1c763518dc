// Matrix-core split-KV kernels for head_dim = 128: one piece per workgroup (single pass, per-sequence chunks).
#include "fdk_splitkv_mfma.h"

namespace fdk {

int launch_splitkv_mfma_d128(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    return launch_mfma_d<128, WM_ONE>(p, q_dtype, kv_dtype, stream);
}

}  // namespace fdk
