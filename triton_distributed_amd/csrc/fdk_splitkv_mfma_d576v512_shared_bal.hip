// Matrix-core split-KV kernels whose wavefronts share the staged tiles (large q-head groups on one kv head), q / K rows
// of 576 values and V rows of 512: balanced mode (equal shares of the whole batch).
#include "fdk_splitkv_mfma_shared.h"

namespace fdk {

int launch_splitkv_mfma_d576v512_shared_bal(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    return launch_mfma_shared<576, 512, WM_SHARES>(p, q_dtype, kv_dtype, stream);
}

}  // namespace fdk
