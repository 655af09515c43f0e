// reduce_copy_inst_f8e5m2.hip -- instantiates the f8e5m2 reduce-copy kernels
// (4 compute ops x n_in 2..8 x aligned/unaligned x temporal/non-temporal, lean and general).
#include "reduce_copy_kernel.h"

namespace pccl_dev {
PCCL_DEFINE_LAUNCH_TYPED(PCCL_F8E5M2)
}  // namespace pccl_dev
