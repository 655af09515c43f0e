// op_graph.h -- the op-DAG layouts under their reference names, and the
// name -> registered-schedule table behind Engine::regOp / exeOp.
//
// RingBuffer, OperationLayoutHeader and GraphBufferLayout are the structs of the
// reference's include/base/operator.h:7-38, byte for byte (static_asserts in
// pccl_op_layout.h); the device kernels read the same definitions.
// OperatorManager is an empty class in the reference (operator.h:40-45).
#pragma once

#include <map>
#include <memory>
#include <mutex>
#include <string>

#include "pccl_op_layout.h"
#include "schedule.h"
#include "type_registry.h"

namespace engine_c {

using RingBuffer = ::pccl_ring_buffer;
using OperationLayoutHeader = ::pccl_operation_layout_header;
using GraphBufferLayout = ::pccl_graph_buffer_layout;

class ExecutorBase;

// A schedule registered under a name, and its device graph once it has been
// bound to buffers.
struct RegisteredOp {
  Schedule schedule;
  std::shared_ptr<ExecutorBase> executor;
  void *graph = nullptr;       // executor graph handle, built at first exeOp
  const void *bound_in = nullptr;
  const void *bound_out = nullptr;
  void *last_stream = nullptr;       // the stream of the latest exeOp
  bool last_stream_known = false;
  ~RegisteredOp();
};

class OperatorManager {
public:
  OperatorManager() = default;
  // Replaces an existing entry of the same name.
  std::shared_ptr<RegisteredOp> add(const std::string &name, Schedule schedule);
  // Throws std::runtime_error for an unknown name.
  std::shared_ptr<RegisteredOp> get(const std::string &name);
  bool has(const std::string &name);
  void remove(const std::string &name);

private:
  std::mutex mu_;
  std::map<std::string, std::shared_ptr<RegisteredOp>> ops_;
};

}  // namespace engine_c
