// graph_queue_inst_f16.hip -- the f16 instances of the drain kernel (one per compute op).
#include "graph_queue_device.h"

namespace pccl_queue {
PCCL_DEFINE_DRAIN_FOR_COMPUTE(PCCL_F16)
}  // namespace pccl_queue
