// graph_queue_fwd_f32.hip -- the f32 instances of the drain kernel that carry the one-pass chain
// code (one per compute op).
#include "graph_queue_device.h"

namespace pccl_queue {
PCCL_DEFINE_DRAIN_FORWARD_FOR_COMPUTE(PCCL_F32)
}  // namespace pccl_queue
