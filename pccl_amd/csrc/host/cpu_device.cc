// cpu_device.cc -- the "cpu" device plugin: host memory for staging, allocated
// as POSIX shared memory like the reference's CpuDevice
// (csrc/plugins/cpu_executor/device.cc:61-95).  Allocator only: the reference's
// shm-name IPC half (device.cc:97-117) hands memory to other processes and is
// not part of this build, and no arithmetic runs on this device.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cstdio>
#include <mutex>
#include <unordered_map>

#include "device_plugin.h"
#include "launch_env.h"

namespace engine_c {

class CpuDevice : public DeviceBase {
public:
  bool allocatorAvailable() override { return true; }

  void *allocate(long nbytes) override {
    if (nbytes <= 0) return nullptr;
    static std::atomic<unsigned long> serial{0};
    char name[96];
    snprintf(name, sizeof(name), "/pccl_amd.%d.%lu", (int)getpid(), serial.fetch_add(1));
    const int fd = shm_open(name, O_CREAT | O_EXCL | O_RDWR, 0600);
    if (fd < 0) return nullptr;
    shm_unlink(name);  // the mapping keeps the memory alive; nothing is left in /dev/shm
    if (ftruncate(fd, nbytes) != 0) {
      close(fd);
      return nullptr;
    }
    void *p = mmap(nullptr, (size_t)nbytes, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    close(fd);
    if (p == MAP_FAILED) return nullptr;
    std::lock_guard<std::mutex> lock(mu_);
    sizes_[p] = nbytes;
    return p;
  }

  void deallocate(void *ptr) override {
    if (!ptr) return;
    std::lock_guard<std::mutex> lock(mu_);
    auto it = sizes_.find(ptr);
    if (it == sizes_.end()) return;
    munmap(ptr, (size_t)it->second);
    sizes_.erase(it);
  }

private:
  std::mutex mu_;
  std::unordered_map<void *, long> sizes_;
};

namespace {
struct CpuPluginRegistration {
  CpuPluginRegistration() {
    const DeviceType device = TypeRegistry::registerDeviceType("cpu");
    regDev(device, std::make_shared<CpuDevice>());
  }
};
static CpuPluginRegistration g_cpu_plugin_registration;
}  // namespace

}  // namespace engine_c
