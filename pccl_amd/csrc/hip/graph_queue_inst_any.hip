// graph_queue_inst_any.hip -- the drain kernel instance that picks dtype and compute op per
// part, for graphs whose REDUCE ops do not share one (dtype, compute) pair.
#include "graph_queue_device.h"

namespace pccl_queue {
DrainKernel drain_for_any() { return drain_graph_kernel<kAnyDtype, void>; }
DrainKernel wide_for_any() { return wide_graph_kernel<kAnyDtype, void>; }
}  // namespace pccl_queue
