// Matrix-core split-KV kernels for head_dim = 128: balanced mode (equal shares of the whole batch).
#include "fdk_splitkv_mfma.h"

namespace fdk {

int launch_splitkv_mfma_d128_bal(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    return launch_mfma_d<128, WM_SHARES>(p, q_dtype, kv_dtype, stream);
}

}  // namespace fdk
