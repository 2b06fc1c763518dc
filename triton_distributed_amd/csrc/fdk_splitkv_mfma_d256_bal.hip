// Matrix-core split-KV kernels for head_dim = 256: balanced mode (equal shares of the whole batch).
#include "fdk_splitkv_mfma.h"

namespace fdk {

int launch_splitkv_mfma_d256_bal(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    return launch_mfma_d<256, WM_SHARES>(p, q_dtype, kv_dtype, stream);
}

}  // namespace fdk
