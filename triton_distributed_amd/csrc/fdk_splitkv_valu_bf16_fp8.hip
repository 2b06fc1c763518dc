// VALU split kernel instantiations: q dtype FDK_BF16, fp8 KV cache: true.
#include "fdk_splitkv_valu_inst.h"

namespace fdk {
namespace valu {
template int launch_typed<FDK_BF16, true>(const SplitParams&, const ValuGeometry&, hipStream_t);
}  // namespace valu
}  // namespace fdk
