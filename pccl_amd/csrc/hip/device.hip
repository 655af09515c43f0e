// device.hip -- device discovery, the allocator and error reporting of
// libpccl_hip.so.  Fills the role of CudaDevice::allocatorAvailable / allocate /
// deallocate (reference csrc/plugins/cuda_executor/device.cc:53-144): sizes are
// rounded up to 2 MiB (:60,70), nbytes <= 0 gives a null pointer (:61), live
// allocations are tracked in a pointer-keyed map under a mutex (:50-51,121-144).
#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "plugin_common.h"

namespace pccl_host {

static thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_error[0] = '\0'; }

int compute_units() {
  static std::mutex mu;
  static std::unordered_map<int, int> cache;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find(dev);
  if (it != cache.end()) return it->second;
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  cache[dev] = cus;
  return cus;
}

// Launch-shape overrides (tuning runs only).  Read on every launch, so lock-free: four relaxed
// atomics, the environment consulted once.
static std::atomic<int> g_tune_wg{0}, g_tune_cache{-1}, g_tune_lds{-1}, g_tune_unroll{-1}, g_tune_rotate{-1};
static std::once_flag g_tuning_env_once;

static void read_tuning_env() {  // same knobs the host plugin lists as launch options
  if (const char *s = getenv("PCCL_HIP_WG_PER_CU")) g_tune_wg.store(atoi(s), std::memory_order_relaxed);
  if (const char *s = getenv("PCCL_HIP_NT")) g_tune_cache.store(std::max(0, std::min(2, atoi(s))), std::memory_order_relaxed);
  if (const char *s = getenv("PCCL_HIP_LDS_BYTES")) g_tune_lds.store(atoi(s), std::memory_order_relaxed);
  if (const char *s = getenv("PCCL_HIP_UNROLL")) g_tune_unroll.store(atoi(s), std::memory_order_relaxed);
  if (const char *s = getenv("PCCL_HIP_ROTATE")) g_tune_rotate.store(atoi(s), std::memory_order_relaxed);
}

Tuning tuning() {
  std::call_once(g_tuning_env_once, read_tuning_env);
  return Tuning{g_tune_wg.load(std::memory_order_relaxed), g_tune_cache.load(std::memory_order_relaxed),
                g_tune_lds.load(std::memory_order_relaxed), g_tune_unroll.load(std::memory_order_relaxed),
                g_tune_rotate.load(std::memory_order_relaxed)};
}

// The id under which the host's TypeRegistry knows this executor (ids are handed out at run time from
// one shared counter, include/base/registry.h:79); written into the executor fields of the device image.
static std::atomic<int> g_executor_id{0};
int executor_id() { return g_executor_id.load(std::memory_order_relaxed); }

// A grid times its 256 lanes must fit 32 bits, so a launch with one workgroup per 4 KiB of every stream
// reaches just under 64 GiB per stream; operands are cut into slices of half that.
static std::atomic<long> g_slice_bytes{32l << 30};
long slice_bytes() { return g_slice_bytes.load(std::memory_order_relaxed); }

// ---- the allocator's bookkeeping -----------------------------------------------------
// One hipMalloc per allocation, the size rounded up to 2 MiB, and a pointer-keyed map of what is
// live under one mutex: what the reference's allocator specifies (cuda_executor/device.cc:50-51,
// 59-70, 121-144).  (An earlier form carved buffers out of 4 GiB blocks and chose their starts by
// the part's memory-channel hash; once the direct kernels rotate the walk over the chunks
// themselves (rotated_chunk, reduce_copy_kernel.h) the same launches ran as fast on plain
// allocations, so that machinery is gone.)
constexpr long kGranule = 2l << 20;

struct Block {
  long bytes;   // as allocated (a multiple of the granule)
  int device;   // the device that holds it
};

static std::mutex g_mem_mutex;
static std::unordered_map<void *, Block> &mem_map() {
  static std::unordered_map<void *, Block> m;
  return m;
}

}  // namespace pccl_host

using namespace pccl_host;

extern "C" {

int pccl_hip_device_count(int *n) {
  clear_error();
  if (!n) return fail(PCCL_ERR_INVALID_ARG, "pccl_hip_device_count: n is null");
  int c = 0;
  hipError_t e = hipGetDeviceCount(&c);
  if (e != hipSuccess) {
    *n = 0;
    (void)hipGetLastError();
    return fail(PCCL_ERR_NO_DEVICE, "hipGetDeviceCount: %s", hipGetErrorString(e));
  }
  *n = c;
  return PCCL_OK;
}

int pccl_hip_device_info(int *cus, long *hbm_bytes, char *name, int name_len) {
  clear_error();
  int dev = 0;
  PCCL_HIP_CHECK(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  PCCL_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
  if (cus) *cus = prop.multiProcessorCount;
  if (hbm_bytes) *hbm_bytes = (long)prop.totalGlobalMem;
  if (name && name_len > 0) {
    snprintf(name, (size_t)name_len, "%s (%s)", prop.name, prop.gcnArchName);
  }
  return PCCL_OK;
}

int pccl_hip_alloc(void **p, long nbytes) {
  clear_error();
  if (!p) return fail(PCCL_ERR_INVALID_ARG, "pccl_hip_alloc: p is null");
  *p = nullptr;
  if (nbytes <= 0) return fail(PCCL_ERR_INVALID_ARG, "pccl_hip_alloc: nbytes %ld <= 0", nbytes);
  const long rounded = (nbytes + kGranule - 1) / kGranule * kGranule;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(PCCL_ERR_NO_DEVICE, "no current device");
  void *q = nullptr;
  const hipError_t e = hipMalloc(&q, (size_t)rounded);
  if (e != hipSuccess || !q) {
    (void)hipGetLastError();
    return fail(PCCL_ERR_NOMEM, "hipMalloc(%ld): %s", rounded, hipGetErrorString(e));
  }
  std::lock_guard<std::mutex> lock(g_mem_mutex);
  mem_map()[q] = Block{rounded, dev};
  *p = q;
  return PCCL_OK;
}

int pccl_hip_free(void *p) {
  clear_error();
  if (!p) return PCCL_OK;
  // The entry leaves the map first: once hipFree has returned, another thread's hipMalloc may be
  // handed the same address.
  Block b;
  {
    std::lock_guard<std::mutex> lock(g_mem_mutex);
    auto it = mem_map().find(p);
    if (it == mem_map().end())
      return fail(PCCL_ERR_INVALID_ARG, "pccl_hip_free: %p was not allocated by pccl_hip_alloc", p);
    b = it->second;
    mem_map().erase(it);
  }
  // hipFree waits for the work that may still use the memory.  It is refused while the calling
  // thread records a stream capture: the buffer then stays allocated, and stays in the map.
  const hipError_t e = hipFree(p);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    std::lock_guard<std::mutex> lock(g_mem_mutex);
    mem_map()[p] = b;
    return fail(PCCL_ERR_HIP, "pccl_hip_free: hipFree(%p): %s (the buffer is still allocated)", p, hipGetErrorString(e));
  }
  return PCCL_OK;
}

int pccl_hip_set_executor_id(int id) {
  clear_error();
  if (id < 0 || id > 255) return fail(PCCL_ERR_INVALID_ARG, "executor id %d does not fit the registry's unsigned char", id);
  g_executor_id.store(id, std::memory_order_relaxed);
  return PCCL_OK;
}

int pccl_hip_set_tuning(int workgroups_per_cu, int cache_treatment) {
  clear_error();
  if (workgroups_per_cu < 0 || workgroups_per_cu > 64)
    return fail(PCCL_ERR_INVALID_ARG, "workgroups_per_cu %d outside [0, 64]", workgroups_per_cu);
  (void)tuning();  // make sure the environment was read before overriding it
  g_tune_wg.store(workgroups_per_cu, std::memory_order_relaxed);
  g_tune_cache.store(cache_treatment < 0 ? -1 : std::min(cache_treatment, 2), std::memory_order_relaxed);
  return PCCL_OK;
}

int pccl_hip_set_unroll(int unroll) {
  clear_error();
  if (unroll != -1 && unroll != 0 && unroll != 1 && unroll != 4)
    return fail(PCCL_ERR_INVALID_ARG, "unroll %d is not -1, 0, 1 or 4", unroll);
  (void)tuning();
  g_tune_unroll.store(unroll, std::memory_order_relaxed);
  return PCCL_OK;
}

int pccl_hip_set_rotation(int rotate) {
  clear_error();
  if (rotate < -1 || rotate > 1) return fail(PCCL_ERR_INVALID_ARG, "rotate %d is not -1, 0 or 1", rotate);
  (void)tuning();
  g_tune_rotate.store(rotate, std::memory_order_relaxed);
  return PCCL_OK;
}

int pccl_hip_set_slice_bytes(long bytes) {
  clear_error();
  if (bytes == 0) bytes = 32l << 30;
  if (bytes < 4096 || bytes % 4096 || bytes > (32l << 30))
    return fail(PCCL_ERR_INVALID_ARG, "slice bytes %ld: not a multiple of 4096 in [4096, 32 GiB]", bytes);
  g_slice_bytes.store(bytes, std::memory_order_relaxed);
  return PCCL_OK;
}

int pccl_hip_set_occupancy_lds(int lds_bytes) {
  clear_error();
  if (lds_bytes > 160 * 1024) return fail(PCCL_ERR_INVALID_ARG, "lds_bytes %d exceeds the 160 KiB of a compute unit", lds_bytes);
  (void)tuning();
  g_tune_lds.store(lds_bytes < 0 ? -1 : lds_bytes, std::memory_order_relaxed);
  return PCCL_OK;
}

const char *pccl_hip_last_error(void) { return g_error; }

int pccl_hip_dtype_bytes(int dtype) { return pccl_dtype_bytes(dtype); }

const char *pccl_hip_version(void) { return "pccl_hip 0.1 (gfx950)"; }

}  // extern "C"
