// reduce_copy_inst_f16.hip -- instantiates the f16 reduce-copy kernels
// (4 compute ops x n_in 2..8 x aligned/unaligned x temporal/non-temporal).
#include "reduce_copy_kernel.h"

namespace pccl_dev {
PCCL_DEFINE_LAUNCH_TYPED(PCCL_F16)
}  // namespace pccl_dev
