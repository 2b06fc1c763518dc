// Matrix-core split-KV kernels for rows of 128 values with more than 16 q heads per kv head (several q-head tiles read the same
// rows: one XCD, plain loads): one piece per workgroup (single pass, per-sequence chunks).
#include "fdk_splitkv_mfma.h"

namespace fdk {

int launch_splitkv_mfma_d128_tiled(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    return launch_mfma_rows2<128, 128, WM_ONE>(p, q_dtype, kv_dtype, stream);
}

}  // namespace fdk
