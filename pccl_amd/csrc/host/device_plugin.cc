#include "device_plugin.h"

#include <map>
#include <mutex>
#include <stdexcept>

namespace engine_c {

namespace {
[[noreturn]] void not_implemented(const char *what) {
  throw std::runtime_error(std::string(what) + " not implemented");
}

struct DeviceTable {
  std::mutex mu;
  std::map<DeviceType, std::shared_ptr<DeviceBase>> devices;
};

// Function-local: plugin translation units call regDev() from their static
// initialisers, in an order the linker chooses.
DeviceTable &table() {
  static DeviceTable *t = new DeviceTable();
  return *t;
}
}  // namespace

bool AllocatorBase::allocatorAvailable() { return false; }
void *AllocatorBase::allocate(long) { not_implemented("AllocatorBase::allocate()"); }
void AllocatorBase::deallocate(void *) { not_implemented("AllocatorBase::deallocate()"); }

bool RemoteCommunicatorBase::remoteCommAvailable() { return false; }
std::string RemoteCommunicatorBase::activate() { not_implemented("RemoteCommunicatorBase::activate()"); }
std::string RemoteCommunicatorBase::regBuffer(void *, long) { not_implemented("RemoteCommunicatorBase::regBuffer()"); }
void RemoteCommunicatorBase::unregBuffer(void *) { not_implemented("RemoteCommunicatorBase::unregBuffer()"); }
void RemoteCommunicatorBase::regRemoteHandle(std::string &) { not_implemented("RemoteCommunicatorBase::regRemoteHandle()"); }
void RemoteCommunicatorBase::connect(std::string) { not_implemented("RemoteCommunicatorBase::connect()"); }
void RemoteCommunicatorBase::disconnect(std::string) { not_implemented("RemoteCommunicatorBase::disconnect()"); }

bool IpcCommunicatorBase::IPCAvailable() { return false; }
std::string IpcCommunicatorBase::registerBuffer(void *, long) { not_implemented("IpcCommunicatorBase::registerBuffer()"); }
std::string IpcCommunicatorBase::allocateIpcBuffer(void **, long) { not_implemented("IpcCommunicatorBase::allocateIpcBuffer()"); }
long IpcCommunicatorBase::mapBuffer(std::string &, void **) { not_implemented("IpcCommunicatorBase::mapBuffer()"); }

std::shared_ptr<DeviceBase> getDev(DeviceType device_type) {
  DeviceTable &t = table();
  std::lock_guard<std::mutex> lock(t.mu);
  auto it = t.devices.find(device_type);
  if (it == t.devices.end())
    throw std::runtime_error("getDev(): no device registered for type " + std::to_string(device_type));
  return it->second;
}

void regDev(DeviceType device_type, std::shared_ptr<DeviceBase> device) {
  DeviceTable &t = table();
  std::lock_guard<std::mutex> lock(t.mu);
  t.devices[device_type] = std::move(device);
}

}  // namespace engine_c
