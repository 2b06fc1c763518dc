// Matrix-core split-KV kernels for rows of 128 values with more than 16 q heads per kv head (several q-head tiles read the same
// rows: one XCD, plain loads): balanced mode (equal shares of the whole batch).
#include "fdk_splitkv_mfma.h"

namespace fdk {

int launch_splitkv_mfma_d128_tiled_bal(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    return launch_mfma_rows2<128, 128, WM_SHARES>(p, q_dtype, kv_dtype, stream);
}

}  // namespace fdk
