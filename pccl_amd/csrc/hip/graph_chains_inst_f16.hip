// graph_chains_inst_f16.hip -- the f16 instances of the kernel that runs a graph of a few independent
// chains as one launch (one per compute op and cache treatment).
#include "graph_chains_device.h"

namespace pccl_queue {
PCCL_DEFINE_CHAINS_FOR_COMPUTE(PCCL_F16)
}  // namespace pccl_queue
