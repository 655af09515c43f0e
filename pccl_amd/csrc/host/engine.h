// engine.h -- Engine: registers compiled collectives by name and runs them.
//
// Method names and roles follow the reference's include/engine.h:13-23 (exposed
// to Python 1:1 by csrc/python_api.cc:13-20).  initEngine() keeps the
// reference's device loop and workspace constants (csrc/engine.cc:15-18,42-100):
// every device type with an allocator gets a 256 MiB workspace followed by 256
// int signal slots, registered with the BufferManager.  regOp() and exeOp() are
// empty / undefined in the reference (csrc/engine.cc:102-104, engine.h:19).
// exeOp() here takes raw device addresses; the at::Tensor form of the reference
// is a two-line wrapper over it (tensor.data_ptr(), tensor.nbytes()).
// exportEndpoint / joinCluster / exitCluster belong to the cluster control plane,
// which this build does not contain; they throw std::runtime_error.
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "chunk_buffers.h"
#include "op_graph.h"

namespace engine_c {

class Engine {
public:
  static constexpr long WORKSPACE_SIZE = 1l << 28;
  static constexpr long GRAN = 1l << 20;
  static constexpr long SLOT = WORKSPACE_SIZE / GRAN;
  static constexpr long TOTAL_SIZE = WORKSPACE_SIZE + SLOT * (long)sizeof(int);

  Engine(int rank, int world_size);
  ~Engine();
  void initEngine();

  // Loads the schedule file at `filepath` (format: schedule.h) under `name`.
  void regOp(const std::string &name, const std::string &filepath);
  // Same, from an in-memory schedule.
  void regOp(const std::string &name, Schedule schedule);

  // Runs the registered collective: `input` and `output` hold the per-device "in" /
  // "out" regions back to back (devices x elems_per_device elements each).  One
  // persistent-kernel launch on `stream`; returns without waiting.
  void exeOp(const std::string &name, const void *input, void *output, long input_bytes, long output_bytes,
             void *stream);
  // Waits for `stream` and checks that every operator of `name` completed.
  void waitOp(const std::string &name, void *stream);

  std::string exportEndpoint();
  void joinCluster(const std::string &master_endpoint);
  void exitCluster();

  BufferManager &buffers() { return *buffers_; }
  OperatorManager &operators() { return *operators_; }
  const std::vector<std::string> &memoryDevices() const { return available_memory_devices_; }
  int rank() const { return rank_; }
  int worldSize() const { return world_size_; }

private:
  int rank_, world_size_;
  std::unique_ptr<BufferManager> buffers_;
  std::unique_ptr<OperatorManager> operators_;
  std::vector<std::string> available_remote_devices_;
  std::vector<std::string> available_memory_devices_;
  std::vector<std::pair<DeviceType, void *>> owned_;
};

}  // namespace engine_c
