// Matrix-core split-KV kernels for q / K rows of 192 values and V rows of 192: per-sequence chunks handed out by a work queue.
#include "fdk_splitkv_mfma.h"

namespace fdk {

int launch_splitkv_mfma_d192_queue(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    return launch_mfma_rows2<192, 192, WM_QUEUE>(p, q_dtype, kv_dtype, stream);
}

}  // namespace fdk
