#include "hip_device.h"

#include <cstdlib>
#include <map>
#include <mutex>
#include <stdexcept>

#include "launch_env.h"
#include "pccl_hip.h"

namespace engine_c {

namespace {

[[noreturn]] void raise(const char *what, int rc) {
  throw std::runtime_error(std::string(what) + " failed (" + std::to_string(rc) + "): " + pccl_hip_last_error());
}

struct CodeTable {
  std::map<GeneralType, int> dtype, compute, primitive;
  ExecutorType executor = 0;
};

CodeTable &codes() {
  static CodeTable *t = new CodeTable();
  return *t;
}

// Self-registration at load time, the reference's plugin idiom
// (csrc/plugins/cuda_executor/device.cc:15-22): device type, then regDev; here
// also the executor, the names it understands, and its launch options
// (csrc/plugins/rdma_executor/device.cc:14-17 registers options the same way).
struct HipPluginRegistration {
  HipPluginRegistration() {
    const DeviceType device = TypeRegistry::registerDeviceType("rocm");
    regDev(device, std::make_shared<HipDevice>());
    CodeTable &t = codes();
    t.executor = TypeRegistry::registerExecutorType("hip");
    (void)pccl_hip_set_executor_id((int)t.executor);  // what the device image's executor fields carry
    const char *prims[] = {"copy", "reduce", "notify", "get_notified"};
    const int prim_codes[] = {PCCL_COPY, PCCL_REDUCE, PCCL_NOTIFY, PCCL_GET_NOTIFIED};
    for (int i = 0; i < 4; ++i) {
      t.primitive[TypeRegistry::registerPrimitive(prims[i])] = prim_codes[i];
      TypeRegistry::registerCompatibility("hip", prims[i]);
    }
    const char *dtypes[] = {"f32", "i32", "bf16", "f16", "f8e4m3", "f8e5m2", "f64", "u32"};
    const int dtype_codes[] = {PCCL_F32, PCCL_I32, PCCL_BF16, PCCL_F16, PCCL_F8E4M3, PCCL_F8E5M2, PCCL_F64, PCCL_U32};
    for (int i = 0; i < PCCL_NUM_DTYPES; ++i) {
      t.dtype[TypeRegistry::registerDataType(dtypes[i])] = dtype_codes[i];
      TypeRegistry::registerCompatibility("hip", dtypes[i]);
    }
    const char *computes[] = {"sum", "prod", "min", "max"};
    const int compute_codes[] = {PCCL_SUM, PCCL_PROD, PCCL_MIN, PCCL_MAX};
    for (int i = 0; i < 4; ++i) {
      t.compute[TypeRegistry::registerComputeType(computes[i])] = compute_codes[i];
      TypeRegistry::registerCompatibility("hip", computes[i]);
    }
    regExecutor(t.executor, std::make_shared<HipExecutor>());
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_WG_PER_CU");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_NT");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_LDS_BYTES");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_UNROLL");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_ROTATE");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_TILE_BYTES");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_PLAN_LAUNCHES");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_PART_DEPS");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_ORDER_BLOCK");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_CHAINS");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_OWN_ENTRIES");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_CHAIN_BALANCE");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_FUSE_SIGNALS");
    utils::LaunchEnvironments::registerOpt("PCCL_HIP_ORDER_EDGES");
  }
};
static HipPluginRegistration g_hip_plugin_registration;

int lookup(const std::map<GeneralType, int> &m, GeneralType id, const char *kind) {
  auto it = m.find(id);
  if (it == m.end())
    throw std::runtime_error(std::string("hip executor: type id ") + std::to_string(id) + " is not a " + kind + " it supports");
  return it->second;
}

struct ExecTable {
  std::mutex mu;
  std::map<ExecutorType, std::shared_ptr<ExecutorBase>> executors;
};
ExecTable &exec_table() {
  static ExecTable *t = new ExecTable();
  return *t;
}

}  // namespace

std::shared_ptr<ExecutorBase> getExecutor(ExecutorType type) {
  ExecTable &t = exec_table();
  std::lock_guard<std::mutex> lock(t.mu);
  auto it = t.executors.find(type);
  if (it == t.executors.end())
    throw std::runtime_error("getExecutor(): no executor registered for type " + std::to_string(type));
  return it->second;
}

std::vector<long> ExecutorBase::carveWorkspace(const void *, long capacity, int n, long nbytes_each) {
  const long stride = (nbytes_each + 255) / 256 * 256;  // every region starts on a 256-byte boundary of the workspace
  if (n < 1 || nbytes_each <= 0 || (long)(n - 1) * stride + nbytes_each > capacity)
    throw std::runtime_error("carveWorkspace(): " + std::to_string(n) + " regions of " + std::to_string(nbytes_each) +
                             " bytes do not fit " + std::to_string(capacity) + " bytes");
  std::vector<long> offsets((size_t)n);
  for (int k = 0; k < n; ++k) offsets[(size_t)k] = (long)k * stride;
  return offsets;
}

void regExecutor(ExecutorType type, std::shared_ptr<ExecutorBase> executor) {
  ExecTable &t = exec_table();
  std::lock_guard<std::mutex> lock(t.mu);
  t.executors[type] = std::move(executor);
}

int hipDtypeCode(DataType id) { return lookup(codes().dtype, id, "data type"); }
int hipComputeCode(ComputeType id) { return lookup(codes().compute, id, "compute type"); }
int hipPrimitiveCode(PrimitiveType id) { return lookup(codes().primitive, id, "primitive"); }

// ---- HipDevice ------------------------------------------------------------------

bool HipDevice::allocatorAvailable() {
  int n = 0;
  return pccl_hip_device_count(&n) == PCCL_OK && n > 0;
}

void *HipDevice::allocate(long nbytes) {
  void *p = nullptr;
  if (pccl_hip_alloc(&p, nbytes) != PCCL_OK) {
    if (nbytes > 0) PCCL_LOG_WARN("HipDevice::allocate(%ld): %s", nbytes, pccl_hip_last_error());
    return nullptr;
  }
  return p;
}

void HipDevice::deallocate(void *ptr) {
  if (!ptr) return;
  const int rc = pccl_hip_free(ptr);
  if (rc != PCCL_OK) PCCL_LOG_WARN("HipDevice::deallocate(%p): %s", ptr, pccl_hip_last_error());
}

// ---- HipExecutor ------------------------------------------------------------------

ExecutorType HipExecutor::type() const { return codes().executor; }

void HipExecutor::reduceCopy(ComputeType compute, const std::vector<ChunkMeta> &ins,
                             const std::vector<ChunkMeta> &outs, void *stream) {
  if (ins.empty() || outs.empty()) throw std::runtime_error("HipExecutor::reduceCopy(): needs inputs and outputs");
  const void *in_ptr[PCCL_MAX_INPUTS];
  void *out_ptr[PCCL_MAX_OUTPUTS];
  if (ins.size() > PCCL_MAX_INPUTS || outs.size() > PCCL_MAX_OUTPUTS)
    throw std::runtime_error("HipExecutor::reduceCopy(): at most 8 inputs and 8 outputs");
  const DataType dt = ins[0].dtype_;
  const long count = ins[0].num_elems_;
  for (size_t k = 0; k < ins.size(); ++k) {
    if (ins[k].dtype_ != dt || ins[k].num_elems_ != count)
      throw std::runtime_error("HipExecutor::reduceCopy(): operands differ in dtype or element count");
    in_ptr[k] = ins[k].addr_;
  }
  for (size_t k = 0; k < outs.size(); ++k) {
    if (outs[k].dtype_ != dt || outs[k].num_elems_ != count)
      throw std::runtime_error("HipExecutor::reduceCopy(): operands differ in dtype or element count");
    out_ptr[k] = outs[k].addr_;
  }
  const int rc = pccl_hip_reduce_copy(hipDtypeCode(dt), hipComputeCode(compute), in_ptr, (int)ins.size(), out_ptr,
                                      (int)outs.size(), count, stream);
  if (rc != PCCL_OK) raise("pccl_hip_reduce_copy", rc);
}

void *HipExecutor::createGraph(const std::vector<BoundOp> &ops) {
  std::vector<pccl_op_desc> descs(ops.size());
  for (size_t i = 0; i < ops.size(); ++i) {
    const BoundOp &o = ops[i];
    pccl_op_desc &d = descs[i];
    d = pccl_op_desc{};
    d.op_uid = (int)i;
    d.primitive = (unsigned char)hipPrimitiveCode(o.primitive);
    const bool is_signal = d.primitive == PCCL_NOTIFY || d.primitive == PCCL_GET_NOTIFIED;
    if (o.ins.size() > PCCL_MAX_INPUTS || o.outs.size() > PCCL_MAX_OUTPUTS || o.ins.size() + o.outs.size() == 0 ||
        (!is_signal && (o.ins.empty() || o.outs.empty())))
      throw std::runtime_error("HipExecutor::createGraph(): op " + std::to_string(i) + " has a bad operand count");
    const ChunkMeta &first = o.ins.empty() ? o.outs[0] : o.ins[0];
    d.dtype = (unsigned char)hipDtypeCode(first.dtype_);
    d.compute = (unsigned char)hipComputeCode(o.compute);
    d.n_in = (unsigned char)o.ins.size();
    d.n_out = (unsigned char)o.outs.size();
    d.count = first.num_elems_;  // signal ops: the value
    for (size_t k = 0; k < o.ins.size(); ++k) d.ins[k] = o.ins[k].addr_;
    for (size_t k = 0; k < o.outs.size(); ++k) d.outs[k] = o.outs[k].addr_;
    d.n_deps = (int)o.deps.size();
    d.deps = o.deps.empty() ? nullptr : o.deps.data();
    if (is_signal) {
      if (o.signal_parts < 0 || o.signal_parts > 0xffff)
        throw std::runtime_error("HipExecutor::createGraph(): op " + std::to_string(i) + " names a signal of " +
                                 std::to_string(o.signal_parts) + " words");
      d.signal_parts = (unsigned short)o.signal_parts;
    }
  }
  // the executor's choice: plain launches for the few graphs that run faster that way, else the queue
  long tile_bytes = PCCL_HIP_TILE_AUTO;
  const std::string tb = utils::LaunchEnvironments::getEnv("PCCL_HIP_TILE_BYTES");
  if (!tb.empty()) {
    char *end = nullptr;
    tile_bytes = strtol(tb.c_str(), &end, 10);
    if (end == tb.c_str() || *end != '\0')
      throw std::runtime_error("HipExecutor::createGraph(): PCCL_HIP_TILE_BYTES='" + tb + "' is not a number of bytes");
  }
  void *graph = nullptr;
  const int rc = pccl_hip_graph_create(descs.data(), (int)descs.size(), tile_bytes, &graph);
  if (rc != PCCL_OK) raise("pccl_hip_graph_create", rc);
  return graph;
}

void HipExecutor::runGraph(void *graph, void *stream) {
  const int rc = pccl_hip_graph_run(graph, stream);
  if (rc != PCCL_OK) raise("pccl_hip_graph_run", rc);
}

std::pair<unsigned, unsigned> HipExecutor::waitGraph(void *graph, void *stream) {
  unsigned done = 0, total = 0;
  const int rc = pccl_hip_graph_status(graph, stream, &done, &total);
  if (rc != PCCL_OK) raise("pccl_hip_graph_status", rc);
  return {done, total};
}

void HipExecutor::rebindGraph(void *graph, const void *old_base, const void *new_base, long nbytes, void *stream) {
  const int rc = pccl_hip_graph_rebind(graph, old_base, new_base, nbytes, stream);
  if (rc != PCCL_OK) raise("pccl_hip_graph_rebind", rc);
}

const GraphBufferLayout *HipExecutor::deviceLayout(void *graph) {
  void *lay = nullptr;
  const int rc = pccl_hip_graph_info(graph, &lay, nullptr, nullptr);
  if (rc != PCCL_OK) raise("pccl_hip_graph_info", rc);
  return static_cast<const GraphBufferLayout *>(lay);
}

void HipExecutor::destroyGraph(void *graph) {
  const int rc = pccl_hip_graph_destroy(graph);
  if (rc != PCCL_OK) PCCL_LOG_WARN("pccl_hip_graph_destroy: %s", pccl_hip_last_error());
}

}  // namespace engine_c
