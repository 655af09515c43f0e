// engine_abi.cc -- extern "C" surface of the host layer (include/pccl_engine.h).
// Catches every exception at the boundary.
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>

#include "device_plugin.h"
#include "engine.h"
#include "executor.h"
#include "hip_device.h"
#include "launch_env.h"
#include "pccl_engine.h"
#include "schedule.h"

using namespace engine_c;

namespace {
thread_local std::string g_error;

template <class F>
int guarded(F &&f) {
  try {
    g_error.clear();
    f();
    return PCCL_ENGINE_OK;
  } catch (const std::exception &e) {
    g_error = e.what();
    return PCCL_ENGINE_ERR;
  } catch (...) {
    g_error = "unknown exception";
    return PCCL_ENGINE_ERR;
  }
}

int bad_arg(const char *what) {
  g_error = what;
  return PCCL_ENGINE_ERR_ARG;
}

void copy_out(const std::string &s, char *buf, int buf_len) {
  if (!buf || buf_len <= 0) throw std::runtime_error("output buffer is null");
  if ((int)s.size() + 1 > buf_len) throw std::runtime_error("output buffer too small");
  memcpy(buf, s.c_str(), s.size() + 1);
}

DeviceType device_id(const char *name) {
  const GeneralType id = TypeRegistry::getTypeId(name);
  if (TypeRegistry::getKind(id) != TypeRegistry::Kind::Device)
    throw std::runtime_error(std::string("'") + name + "' is not a device type");
  return id;
}
}  // namespace

extern "C" {

int pccl_engine_create(int rank, int world_size, void **engine) {
  if (!engine) return bad_arg("engine is null");
  *engine = nullptr;
  return guarded([&] { *engine = new Engine(rank, world_size); });
}

int pccl_engine_destroy(void *engine) {
  return guarded([&] { delete static_cast<Engine *>(engine); });
}

int pccl_engine_init(void *engine) {
  if (!engine) return bad_arg("engine is null");
  return guarded([&] { static_cast<Engine *>(engine)->initEngine(); });
}

int pccl_engine_reg_op(void *engine, const char *name, const char *filepath) {
  if (!engine || !name || !filepath) return bad_arg("null argument");
  return guarded([&] { static_cast<Engine *>(engine)->regOp(std::string(name), std::string(filepath)); });
}

int pccl_engine_reg_op_text(void *engine, const char *name, const char *text) {
  if (!engine || !name || !text) return bad_arg("null argument");
  return guarded([&] { static_cast<Engine *>(engine)->regOp(std::string(name), Schedule::parse(text)); });
}

int pccl_engine_exe_op(void *engine, const char *name, const void *input, long input_bytes, void *output,
                       long output_bytes, void *stream) {
  if (!engine || !name) return bad_arg("null argument");
  return guarded([&] { static_cast<Engine *>(engine)->exeOp(name, input, output, input_bytes, output_bytes, stream); });
}

int pccl_engine_wait_op(void *engine, const char *name, void *stream) {
  if (!engine || !name) return bad_arg("null argument");
  return guarded([&] { static_cast<Engine *>(engine)->waitOp(name, stream); });
}

int pccl_engine_get_dev_buffer(void *engine, const char *device_name, void **workspace, void **signals,
                               long *workspace_bytes) {
  if (!engine || !device_name) return bad_arg("null argument");
  return guarded([&] {
    Engine *e = static_cast<Engine *>(engine);
    const DeviceType id = device_id(device_name);
    auto [ws, sig] = e->buffers().getDevBuffer(id);
    if (workspace) *workspace = ws;
    if (signals) *signals = sig;
    if (workspace_bytes) *workspace_bytes = e->buffers().getDevBufferSize(id);
  });
}

int pccl_engine_op_info(void *engine, const char *name, int *n_ops, int *devices, long *elems_per_device,
                        int *elem_bytes) {
  if (!engine || !name) return bad_arg("null argument");
  return guarded([&] {
    auto op = static_cast<Engine *>(engine)->operators().get(name);
    if (n_ops) *n_ops = (int)op->schedule.ops.size();
    if (devices) *devices = op->schedule.devices;
    if (elems_per_device) *elems_per_device = op->schedule.elems_per_device;
    if (elem_bytes) *elem_bytes = op->schedule.elemBytes();
  });
}

int pccl_engine_export_endpoint(void *engine, char *buf, int buf_len) {
  if (!engine) return bad_arg("engine is null");
  return guarded([&] { copy_out(static_cast<Engine *>(engine)->exportEndpoint(), buf, buf_len); });
}

int pccl_engine_join_cluster(void *engine, const char *master_endpoint) {
  if (!engine || !master_endpoint) return bad_arg("null argument");
  return guarded([&] { static_cast<Engine *>(engine)->joinCluster(master_endpoint); });
}

int pccl_engine_exit_cluster(void *engine) {
  if (!engine) return bad_arg("engine is null");
  return guarded([&] { static_cast<Engine *>(engine)->exitCluster(); });
}

int pccl_engine_reduce_copy(const char *dtype, const char *compute, const void *const *ins, int n_in,
                            void *const *outs, int n_out, long count, void *stream) {
  if (!dtype || !compute || !ins || !outs) return bad_arg("null argument");
  return guarded([&] {
    if (n_in < 1 || n_in > 8 || n_out < 1 || n_out > 8) throw std::runtime_error("n_in / n_out outside [1, 8]");
    const DataType dt = TypeRegistry::getTypeId(dtype);
    const ComputeType op = TypeRegistry::getTypeId(compute);
    std::vector<ChunkMeta> i, o;
    for (int k = 0; k < n_in; ++k) i.push_back(ChunkMeta{dt, const_cast<void *>(ins[k]), count});
    for (int k = 0; k < n_out; ++k) o.push_back(ChunkMeta{dt, outs[k], count});
    getExecutor(TypeRegistry::getTypeId("hip"))->reduceCopy(op, i, o, stream);
  });
}

int pccl_registry_type_id(const char *name, int *id) {
  if (!name || !id) return bad_arg("null argument");
  return guarded([&] { *id = TypeRegistry::getTypeId(name); });
}

int pccl_registry_type_name(int id, char *buf, int buf_len) {
  return guarded([&] {
    if (id < 0 || id > 255) throw std::out_of_range("type id outside [0, 255]");
    copy_out(std::string(TypeRegistry::getTypeName((GeneralType)id)), buf, buf_len);
  });
}

int pccl_registry_register(int kind, const char *name, int *id) {
  if (!name) return bad_arg("name is null");
  return guarded([&] {
    GeneralType r;
    switch (kind) {
      case 0: r = TypeRegistry::registerPrimitive(name); break;
      case 1: r = TypeRegistry::registerDataType(name); break;
      case 2: r = TypeRegistry::registerComputeType(name); break;
      case 3: r = TypeRegistry::registerDeviceType(name); break;
      case 4: r = TypeRegistry::registerExecutorType(name); break;
      default: throw std::runtime_error("kind outside [0, 4]");
    }
    if (id) *id = r;
  });
}

int pccl_registry_register_compat(const char *executor, const char *type_name) {
  if (!executor || !type_name) return bad_arg("null argument");
  return guarded([&] { TypeRegistry::registerCompatibility(executor, type_name); });
}

int pccl_registry_is_compatible(const char *executor, const char *type_name, int *yes) {
  if (!executor || !type_name || !yes) return bad_arg("null argument");
  return guarded([&] {
    const auto &set = TypeRegistry::getCompatibleTypes(TypeRegistry::getTypeId(executor));
    *yes = set.count(TypeRegistry::getTypeId(type_name)) ? 1 : 0;
  });
}

int pccl_registry_device_types(char *buf, int buf_len) {
  return guarded([&] {
    std::string s;
    for (DeviceType d : TypeRegistry::getDeviceTypes()) {
      if (!s.empty()) s += '\n';
      s += std::string(TypeRegistry::getTypeName(d));
    }
    copy_out(s, buf, buf_len);
  });
}

int pccl_device_allocator_available(const char *device_name, int *yes) {
  if (!device_name || !yes) return bad_arg("null argument");
  return guarded([&] { *yes = getDev(device_id(device_name))->allocatorAvailable() ? 1 : 0; });
}

int pccl_device_allocate(const char *device_name, long nbytes, void **p) {
  if (!device_name || !p) return bad_arg("null argument");
  return guarded([&] { *p = getDev(device_id(device_name))->allocate(nbytes); });
}

int pccl_device_deallocate(const char *device_name, void *p) {
  if (!device_name) return bad_arg("null argument");
  return guarded([&] { getDev(device_id(device_name))->deallocate(p); });
}

int pccl_device_ipc_available(const char *device_name, int *yes) {
  if (!device_name || !yes) return bad_arg("null argument");
  return guarded([&] { *yes = getDev(device_id(device_name))->IPCAvailable() ? 1 : 0; });
}

int pccl_env_list_opt(char *buf, int buf_len) {
  return guarded([&] {
    std::string s;
    for (const std::string &o : utils::LaunchEnvironments::listOpt()) {
      if (!s.empty()) s += '\n';
      s += o;
    }
    copy_out(s, buf, buf_len);
  });
}

int pccl_env_get(const char *name, char *buf, int buf_len) {
  if (!name) return bad_arg("name is null");
  return guarded([&] { copy_out(utils::LaunchEnvironments::getEnv(name), buf, buf_len); });
}

int pccl_env_register_opt(const char *name) {
  if (!name) return bad_arg("name is null");
  return guarded([&] { utils::LaunchEnvironments::registerOpt(name); });
}

int pccl_schedule_write_ring_allreduce(const char *path, const char *dtype, const char *compute, int devices,
                                       long chunk_elems) {
  if (!path || !dtype || !compute) return bad_arg("null argument");
  return guarded([&] {
    if (devices < 1 || chunk_elems < 0) throw std::runtime_error("devices must be >= 1 and chunk_elems >= 0");
    Schedule s;
    s.name = "ring_allreduce";
    s.dtype = dtype;
    s.compute = compute;
    s.devices = devices;
    appendRingAllReduce(s, chunk_elems, 0);
    s.validate();
    s.save(path);
  });
}

int pccl_schedule_write_direct_allreduce(const char *path, const char *dtype, const char *compute, int devices,
                                         long slice_elems) {
  if (!path || !dtype || !compute) return bad_arg("null argument");
  return guarded([&] {
    if (devices < 1 || slice_elems < 0) throw std::runtime_error("devices must be >= 1 and slice_elems >= 0");
    Schedule s;
    s.name = "direct_allreduce";
    s.dtype = dtype;
    s.compute = compute;
    s.devices = devices;
    appendDirectAllReduce(s, slice_elems, 0);
    s.validate();
    s.save(path);
  });
}

int pccl_schedule_write_collective(const char *path, const char *kind, const char *dtype, const char *compute,
                                   int devices, long elems, int root) {
  if (!path || !kind || !dtype || !compute) return bad_arg("null argument");
  return guarded([&] {
    if (devices < 1 || elems < 0) throw std::runtime_error("devices must be >= 1 and elems >= 0");
    Schedule s;
    s.name = kind;
    s.dtype = dtype;
    s.compute = compute;
    s.devices = devices;
    const std::string k = kind;
    if (k == "ring_allreduce") appendRingAllReduce(s, elems, 0);
    else if (k == "direct_allreduce") appendDirectAllReduce(s, elems, 0);
    else if (k == "ring_reduce_scatter") appendRingReduceScatter(s, elems, 0);
    else if (k == "ring_all_gather") appendRingAllGather(s, elems, 0);
    else if (k == "broadcast") appendBroadcast(s, elems, root, 0);
    else if (k == "all_to_all") appendAllToAll(s, elems, 0);
    else throw std::runtime_error("unknown collective '" + k + "'");
    s.validate();
    s.save(path);
  });
}

int pccl_schedule_write_small_message(const char *path, const char *dtype, int devices, int n_slices, int n_extra,
                                      unsigned long seed, long lo_bytes, long hi_bytes) {
  if (!path || !dtype) return bad_arg("null argument");
  return guarded([&] {
    if (devices < 1 || n_slices < 0 || n_extra < 0 || lo_bytes < 1 || hi_bytes < lo_bytes)
      throw std::runtime_error("bad small-message schedule parameters");
    makeSmallMessageSchedule(devices, n_slices, n_extra, seed, lo_bytes, hi_bytes, dtype).save(path);
  });
}

int pccl_schedule_inspect(const char *path, int *n_ops, int *devices, long *elems_per_device, int *order,
                          int order_len) {
  if (!path) return bad_arg("path is null");
  return guarded([&] {
    const Schedule s = Schedule::load(path);
    if (n_ops) *n_ops = (int)s.ops.size();
    if (devices) *devices = s.devices;
    if (elems_per_device) *elems_per_device = s.elems_per_device;
    if (order) {
      if (order_len < (int)s.ops.size()) throw std::runtime_error("order buffer too small");
      const std::vector<int> o = s.topologicalOrder();
      for (size_t i = 0; i < o.size(); ++i) order[i] = o[i];
    }
  });
}

const char *pccl_engine_last_error(void) { return g_error.c_str(); }

}  // extern "C"
