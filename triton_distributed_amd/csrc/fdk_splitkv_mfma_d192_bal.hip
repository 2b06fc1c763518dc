// Matrix-core split-KV kernels for q / K rows of 192 values and V rows of 192: balanced mode (equal shares of the whole batch).
#include "fdk_splitkv_mfma.h"

namespace fdk {

int launch_splitkv_mfma_d192_bal(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    return launch_mfma_rows2<192, 192, WM_SHARES>(p, q_dtype, kv_dtype, stream);
}

}  // namespace fdk
