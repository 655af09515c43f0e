#include "engine.h"

#include <algorithm>
#include <exception>
#include <stdexcept>

#include "device_plugin.h"
#include "executor.h"
#include "launch_env.h"

namespace engine_c {

Engine::Engine(int rank, int world_size) : rank_(rank), world_size_(world_size) {
  if (world_size < 1 || rank < 0 || rank >= world_size)
    throw std::runtime_error("Engine: rank " + std::to_string(rank) + " outside world of " + std::to_string(world_size));
}

Engine::~Engine() {
  operators_.reset();  // graphs first: they hold device memory of their own
  for (auto &[type, ptr] : owned_) {
    try {
      getDev(type)->deallocate(ptr);
    } catch (const std::exception &e) {
      PCCL_LOG_WARN("Engine: releasing a workspace failed: %s", e.what());
    }
  }
}

void Engine::initEngine() {
  if (buffers_) throw std::runtime_error("Engine::initEngine(): already initialised");
  buffers_ = std::make_unique<BufferManager>();
  operators_ = std::make_unique<OperatorManager>();
  available_remote_devices_.clear();
  available_memory_devices_.clear();
  for (DeviceType device : TypeRegistry::getDeviceTypes()) {
    const std::string device_name(TypeRegistry::getTypeName(device));
    auto dev = getDev(device);
    // No plugin of this build offers remote communication or IPC, so the
    // reference's first two branches (csrc/engine.cc:56-73) are never taken.
    if (dev->remoteCommAvailable()) available_remote_devices_.push_back(device_name);
    if (!dev->allocatorAvailable()) continue;
    void *buffer = dev->allocate(TOTAL_SIZE);
    if (!buffer) {
      PCCL_LOG_WARN("Engine::initEngine(): device '%s' could not allocate its workspace", device_name.c_str());
      continue;
    }
    owned_.push_back({device, buffer});
    int *signal_buffer = reinterpret_cast<int *>(static_cast<char *>(buffer) + WORKSPACE_SIZE);
    buffers_->regBuffer(buffer, WORKSPACE_SIZE, signal_buffer, SLOT, rank_, device);
    available_memory_devices_.push_back(device_name);
  }
}

void Engine::regOp(const std::string &name, const std::string &filepath) { regOp(name, Schedule::load(filepath)); }

void Engine::regOp(const std::string &name, Schedule schedule) {
  if (!operators_) throw std::runtime_error("Engine::regOp(): call initEngine() first");
  schedule.validate();
  // every name the schedule uses must be known to the registry and runnable by the hip executor
  const ExecutorType hip = TypeRegistry::getTypeId("hip");
  const auto &ok = TypeRegistry::getCompatibleTypes(hip);
  for (const std::string &n : {schedule.dtype, schedule.compute})
    if (!TypeRegistry::hasType(n) || !ok.count(TypeRegistry::getTypeId(n)))
      throw std::runtime_error("Engine::regOp(): executor 'hip' does not support '" + n + "'");
  auto op = operators_->add(name, std::move(schedule));
  op->executor = getExecutor(hip);
}

void Engine::exeOp(const std::string &name, const void *input, void *output, long input_bytes, long output_bytes,
                   void *stream) {
  if (!operators_) throw std::runtime_error("Engine::exeOp(): call initEngine() first");
  auto op = operators_->get(name);
  const Schedule &s = op->schedule;
  const long es = s.elemBytes();
  const long need = (long)s.devices * s.elems_per_device * es;
  if (!input || !output) throw std::runtime_error("Engine::exeOp(): null tensor");
  if (input_bytes < need || output_bytes < need)
    throw std::runtime_error("Engine::exeOp(): '" + name + "' needs " + std::to_string(need) +
                             " bytes per tensor, got " + std::to_string(input_bytes) + " / " + std::to_string(output_bytes));
  // One graph runs one launch at a time: a run that an earlier call started on another stream ends
  // before this call rebinds, rebuilds or runs the graph again (same stream: stream order does it).
  if (op->graph && op->last_stream_known && op->last_stream != stream) {
    try {
      op->executor->waitGraph(op->graph, op->last_stream);
    } catch (...) {
      // reported once (that run gave up, or its stream no longer exists); the op stays usable
      op->last_stream_known = false;
      throw;
    }
  }
  if (!op->graph) {
    const DeviceType rocm = TypeRegistry::getTypeId("rocm");
    char *ws = nullptr;
    long ws_bytes = 0;
    if (buffers_->hasDevBuffer(rocm)) {
      ws = static_cast<char *>(std::get<0>(buffers_->getDevBuffer(rocm)));
      ws_bytes = buffers_->getDevBufferSize(rocm);
    }
    const DataType dt = TypeRegistry::getTypeId(s.dtype);
    const ComputeType compute = TypeRegistry::getTypeId(s.compute);
    const PrimitiveType copy = TypeRegistry::getTypeId("copy"), reduce = TypeRegistry::getTypeId("reduce");
    // "ws" operands live in per-device regions of the workspace, each as large as the schedule needs,
    // laid out by the executor (back to back, each on a 256-byte boundary)
    long ws_need = 0;
    for (const ScheduleOp &o : s.ops) {
      if (o.isSignal()) continue;
      for (const auto &x : o.srcs) if (x.buffer == "ws") ws_need = std::max(ws_need, (x.offset + o.count) * es);
      for (const auto &x : o.dsts) if (x.buffer == "ws") ws_need = std::max(ws_need, (x.offset + o.count) * es);
    }
    std::vector<long> ws_region;
    if (ws_need > 0) {
      if (!ws) throw std::runtime_error("Engine::exeOp(): the schedule uses the workspace, but no device has one");
      try {
        ws_region = op->executor->carveWorkspace(ws, ws_bytes, s.devices, ws_need);
      } catch (const std::exception &e) {
        throw std::runtime_error(std::string("Engine::exeOp(): workspace operand does not fit the device workspace: ") + e.what());
      }
    }
    auto resolve = [&](const ScheduleOperand &x, long count) -> void * {
      (void)count;
      if (x.buffer == "ws") return ws + ws_region[(size_t)x.device] + x.offset * es;
      const char *base = x.buffer == "in" ? static_cast<const char *>(input) : static_cast<char *>(output);
      return const_cast<char *>(base) + ((long)x.device * s.elems_per_device + x.offset) * es;
    };
    const PrimitiveType notify = TypeRegistry::getTypeId("notify"), get_notified = TypeRegistry::getTypeId("get_notified");
    int *signals = nullptr;
    if (buffers_->hasDevBuffer(rocm)) signals = static_cast<int *>(std::get<1>(buffers_->getDevBuffer(rocm)));
    std::vector<BoundOp> bound(s.ops.size());
    for (size_t i = 0; i < s.ops.size(); ++i) {
      const ScheduleOp &o = s.ops[i];
      BoundOp &b = bound[i];
      if (o.isSignal()) {  // the operand is one of the workspace's signal slots, the count its value
        if (!signals || o.slot + o.parts > SLOT)
          throw std::runtime_error("Engine::exeOp(): signal slot " + std::to_string(o.slot) + " is not available");
        b.signal_parts = o.parts;
        b.primitive = o.kind == ScheduleOp::NOTIFY ? notify : get_notified;
        b.compute = compute;
        b.deps = o.deps;
        const ChunkMeta word{dt, signals + o.slot, o.count};
        (o.kind == ScheduleOp::NOTIFY ? b.outs : b.ins).push_back(word);
        continue;
      }
      b.primitive = o.reduce ? reduce : copy;
      b.compute = compute;
      b.deps = o.deps;
      for (const auto &x : o.srcs) b.ins.push_back(ChunkMeta{dt, resolve(x, o.count), o.count});
      for (const auto &x : o.dsts) b.outs.push_back(ChunkMeta{dt, resolve(x, o.count), o.count});
    }
    op->graph = op->executor->createGraph(bound);
    op->bound_in = input;
    op->bound_out = output;
  } else if (op->bound_in != input || op->bound_out != output) {
    // New tensors.  Moving operands range by range is only safe when no new range
    // touches an old one (an operand must not be moved twice); otherwise rebuild.
    auto apart = [need](const void *a, const void *b) {
      const char *x = static_cast<const char *>(a), *y = static_cast<const char *>(b);
      return x + need <= y || y + need <= x;
    };
    const bool in_moves = op->bound_in != input, out_moves = op->bound_out != output;
    const bool safe = apart(op->bound_in, op->bound_out) && apart(input, output) &&
                      (!in_moves || (apart(input, op->bound_in) && apart(input, op->bound_out))) &&
                      (!out_moves || (apart(output, op->bound_out) && apart(output, op->bound_in)));
    bool rebuild = !safe;
    if (safe) {
      try {
        if (in_moves) {
          op->executor->rebindGraph(op->graph, op->bound_in, input, need, stream);
          op->bound_in = input;
        }
        if (out_moves) {
          op->executor->rebindGraph(op->graph, op->bound_out, output, need, stream);
          op->bound_out = output;
        }
      } catch (const std::exception &e) {
        // (the executor cannot move this graph's operands, or moved only half of them: build it again)
        PCCL_LOG_WARN("Engine::exeOp(): '%s' is built again for its new tensors: %s", name.c_str(), e.what());
        rebuild = true;
      }
    }
    if (rebuild) {
      // The graph's device state goes away: the stream it may still be running on ends first.  If that
      // run gave up, this call reports it (once); the graph is gone either way and the next call builds it.
      std::exception_ptr gave_up;
      try {
        op->executor->waitGraph(op->graph, stream);
      } catch (...) {
        gave_up = std::current_exception();
      }
      op->executor->destroyGraph(op->graph);
      op->graph = nullptr;
      op->last_stream_known = false;
      if (gave_up) std::rethrow_exception(gave_up);
      exeOp(name, input, output, input_bytes, output_bytes, stream);
      return;
    }
  }
  op->executor->runGraph(op->graph, stream);
  op->last_stream = stream;
  op->last_stream_known = true;
}

void Engine::waitOp(const std::string &name, void *stream) {
  auto op = operators_->get(name);
  if (!op->graph) return;
  const auto [done, total] = op->executor->waitGraph(op->graph, stream);
  if (done != total)
    throw std::runtime_error("Engine::waitOp(): '" + name + "' completed " + std::to_string(done) + " of " +
                             std::to_string(total) + " operators");
}

std::string Engine::exportEndpoint() { throw std::runtime_error("Engine::exportEndpoint(): no cluster control plane in this build"); }
void Engine::joinCluster(const std::string &) { throw std::runtime_error("Engine::joinCluster(): no cluster control plane in this build"); }
void Engine::exitCluster() { throw std::runtime_error("Engine::exitCluster(): no cluster control plane in this build"); }

}  // namespace engine_c
