// graph_queue_fwd_f8e4m3.hip -- the f8e4m3 instances of the drain kernel that carry the one-pass chain
// code (one per compute op).
#include "graph_queue_device.h"

namespace pccl_queue {
PCCL_DEFINE_DRAIN_FORWARD_FOR_COMPUTE(PCCL_F8E4M3)
}  // namespace pccl_queue
