// Split-KV paged GQA decode, matrix-core path.  (Not built yet: the planner never selects it.)
#include "fdk_device.h"

namespace fdk {

bool mfma_supported(int, int, int) { return false; }
int mfma_heads_per_wg(int) { return 16; }
int launch_splitkv_mfma(const SplitParams&, int, int, hipStream_t) { return (int)hipErrorNotSupported; }

}  // namespace fdk
