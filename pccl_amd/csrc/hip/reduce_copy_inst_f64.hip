// reduce_copy_inst_f64.hip -- instantiates the f64 reduce-copy kernels
// (4 compute ops x n_in 2..8 x aligned/unaligned x cache treatment, lean and general).
#include "reduce_copy_kernel.h"

namespace pccl_dev {
PCCL_DEFINE_LAUNCH_TYPED(PCCL_F64)
}  // namespace pccl_dev
