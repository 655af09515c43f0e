// hip_device.h -- the MI355X device plugin ("rocm") and its executor ("hip").
//
// HipDevice takes the place of the reference's CudaDevice
// (include/plugins/cuda_executor/device.h:7-16,
// csrc/plugins/cuda_executor/device.cc:53-144): allocator methods only.  The IPC
// methods of CudaDevice (device.cc:146-196) export memory to other processes and
// stay at the base-class behaviour (IPCAvailable() == false).
// Both classes talk to the GPU only through the C ABI of libpccl_hip.so.
#pragma once

#include "device_plugin.h"
#include "executor.h"

namespace engine_c {

class HipDevice : public DeviceBase {
public:
  bool allocatorAvailable() override;
  void *allocate(long nbytes) override;   // nullptr on failure or nbytes <= 0, like cuda device.cc:61,74-119
  void deallocate(void *ptr) override;
};

class HipExecutor : public ExecutorBase {
public:
  ExecutorType type() const override;
  void reduceCopy(ComputeType compute, const std::vector<ChunkMeta> &ins, const std::vector<ChunkMeta> &outs,
                  void *stream) override;
  void *createGraph(const std::vector<BoundOp> &ops) override;
  void runGraph(void *graph, void *stream) override;
  std::pair<unsigned, unsigned> waitGraph(void *graph, void *stream) override;
  void rebindGraph(void *graph, const void *old_base, const void *new_base, long nbytes, void *stream) override;
  const GraphBufferLayout *deviceLayout(void *graph) override;
  void destroyGraph(void *graph) override;
};

// Registry id -> code of include/pccl_hip.h; throws std::runtime_error for an id
// the hip executor is not compatible with.
int hipDtypeCode(DataType id);
int hipComputeCode(ComputeType id);
int hipPrimitiveCode(PrimitiveType id);

}  // namespace engine_c
