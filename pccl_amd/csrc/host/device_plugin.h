// device_plugin.h -- the plugin interface a device type implements, and the
// process-wide device table.
//
// Same three mix-ins and the same method names as the reference's
// include/base/device.h:8-43.  A method a plugin does not override behaves like
// the reference's base (csrc/base/device.cc:10-62): the availability probes
// answer false, every other call throws
// std::runtime_error("<Class>::<method>() not implemented").
// getDev() returns the registered plugin (the reference's always throws,
// csrc/base/device.cc:65-67) and throws std::runtime_error for an unknown type.
#pragma once

#include <memory>
#include <string>

#include "type_registry.h"

namespace engine_c {

class AllocatorBase {
public:
  virtual ~AllocatorBase() = default;
  virtual bool allocatorAvailable();
  virtual void *allocate(long nbytes);
  virtual void deallocate(void *ptr);
};

class RemoteCommunicatorBase {
public:
  virtual ~RemoteCommunicatorBase() = default;
  virtual bool remoteCommAvailable();
  virtual std::string activate();
  virtual std::string regBuffer(void *addr, long size);
  virtual void unregBuffer(void *addr);
  virtual void regRemoteHandle(std::string &handle);
  virtual void connect(std::string handle);
  virtual void disconnect(std::string handle);
};

class IpcCommunicatorBase {
public:
  virtual ~IpcCommunicatorBase() = default;
  virtual bool IPCAvailable();
  virtual std::string registerBuffer(void *addr, long size);
  virtual std::string allocateIpcBuffer(void **addr, long size);
  virtual long mapBuffer(std::string &shareable_handle, void **addr);
};

class DeviceBase : public AllocatorBase, public RemoteCommunicatorBase, public IpcCommunicatorBase {};

std::shared_ptr<DeviceBase> getDev(DeviceType device_type);
void regDev(DeviceType device_type, std::shared_ptr<DeviceBase> device);

}  // namespace engine_c
