// reduce_copy_inst_f8e4m3.hip -- instantiates the f8e4m3 reduce-copy kernels
// (4 compute ops x n_in 2..8 x aligned/unaligned x temporal/non-temporal, lean and general).
#include "reduce_copy_kernel.h"

namespace pccl_dev {
PCCL_DEFINE_LAUNCH_TYPED(PCCL_F8E4M3)
}  // namespace pccl_dev
