// executor.h -- what an executor plugin offers the engine: run one reduce-copy,
// and hold / run whole op graphs.
//
// The reference reserves include/plugins/cuda_executor/executor.h and
// include/plugins/cpu_executor/executor.h for this and leaves both empty, so
// the interface is defined here.  Operands are ChunkMeta
// (include/base/chunk.h:10-14); type arguments are TypeRegistry ids.
#pragma once

#include <memory>
#include <vector>

#include "chunk_buffers.h"
#include "op_graph.h"

namespace engine_c {

// One IR operation with operands resolved to addresses.
struct BoundOp {
  PrimitiveType primitive;  // registry id of "copy" / "reduce"
  ComputeType compute;      // registry id of "sum" / "prod" / "min" / "max"
  std::vector<ChunkMeta> ins;
  std::vector<ChunkMeta> outs;
  std::vector<int> deps;    // indices of ops that must complete first
  int signal_parts = 0;     // NOTIFY / GET_NOTIFIED: words of the signal, one per part of the data it announces (0, 1: one word)
};

class ExecutorBase {
public:
  virtual ~ExecutorBase() = default;
  virtual ExecutorType type() const = 0;

  // outs[j][i] = fold(compute, ins[0][i], ..., ins[n-1][i]); asynchronous on `stream`.
  virtual void reduceCopy(ComputeType compute, const std::vector<ChunkMeta> &ins,
                          const std::vector<ChunkMeta> &outs, void *stream) = 0;

  // Graph handles are opaque; the executor owns what they point to.
  virtual void *createGraph(const std::vector<BoundOp> &ops) = 0;
  virtual void runGraph(void *graph, void *stream) = 0;
  // Waits for `stream`; returns (completed, total) operators.
  virtual std::pair<unsigned, unsigned> waitGraph(void *graph, void *stream) = 0;
  virtual void rebindGraph(void *graph, const void *old_base, const void *new_base, long nbytes, void *stream) = 0;
  virtual const GraphBufferLayout *deviceLayout(void *graph) = 0;
  virtual void destroyGraph(void *graph) = 0;

  // Byte offsets of n regions of nbytes_each inside [base, base + capacity): how the executor wants a
  // workspace divided among the devices of a schedule (the role of BufferManager::assignBuffer,
  // include/base/chunk.h:48-53).  Throws std::runtime_error when they do not fit.
  // Default: back to back, each region on a 256-byte boundary.
  virtual std::vector<long> carveWorkspace(const void *base, long capacity, int n, long nbytes_each);
};

std::shared_ptr<ExecutorBase> getExecutor(ExecutorType type);
void regExecutor(ExecutorType type, std::shared_ptr<ExecutorBase> executor);

}  // namespace engine_c
