// Contiguous-row kernels instantiated for one storage type.
#include "rows_launch_impl.hip.h"

namespace atexn {
ATEXN_INSTANTIATE_ROWS(bf16_t)
}  // namespace atexn
