// Channels-last InstanceNorm kernels instantiated for the three storage types.
#include "cl_launch_impl.hip.h"

namespace atexn {
ATEXN_INSTANTIATE_CL(float)
ATEXN_INSTANTIATE_CL(f16_t)
ATEXN_INSTANTIATE_CL(bf16_t)
}  // namespace atexn
