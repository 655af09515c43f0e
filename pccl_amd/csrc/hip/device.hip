// device.hip -- device discovery, the allocator and error reporting of
// libpccl_hip.so.  Fills the role of CudaDevice::allocatorAvailable / allocate /
// deallocate (reference csrc/plugins/cuda_executor/device.cc:53-144): sizes are
// rounded up to 2 MiB (:60,70), nbytes <= 0 gives a null pointer (:61), live
// allocations are tracked in a pointer-keyed map under a mutex (:50-51,121-144).
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>

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

static std::mutex g_tuning_mutex;
static Tuning g_tuning = {0, -1, -1, -1};
static bool g_tuning_env_read = false;

Tuning tuning() {
  std::lock_guard<std::mutex> lock(g_tuning_mutex);
  if (!g_tuning_env_read) {  // same knobs the host plugin lists as launch options
    g_tuning_env_read = true;
    if (const char *s = getenv("PCCL_HIP_WG_PER_CU")) g_tuning.workgroups_per_cu = atoi(s);
    if (const char *s = getenv("PCCL_HIP_NT")) g_tuning.cache_treatment = std::max(0, std::min(2, atoi(s)));
    if (const char *s = getenv("PCCL_HIP_LDS_BYTES")) g_tuning.lds_bytes = atoi(s);
    if (const char *s = getenv("PCCL_HIP_UNROLL")) g_tuning.unroll = atoi(s);
  }
  return g_tuning;
}

// Distance added between the buffers of a group when the caller leaves the choice open.
// Measured with bf16 reductions on group allocations (TB/s at pad 0 -> at this pad): 8 -> 1 at
// 256 MiB 6.5 -> 6.8, at 128 MiB 6.6 -> 6.75, 8 -> 2 at 128 MiB 6.65 -> 6.9, 2 -> 2 at 32 MiB
// 7.1 -> 7.1.  Pads of 4-68 KiB help the 256 MiB case as much but cost the 128 MiB cases 10 %,
// and 1028 KiB does the opposite, so the effect is not monotonic in the pad.
constexpr long kDefaultGroupPad = (576l << 10) + 4096;
// Below about 96 MiB per buffer that pad costs (8 -> 1 at 64 MiB: 6.8 -> 5.6-6.3) where a small one
// is neutral or helps (8 -> 1 at 64 MiB 6.8 -> 6.85, 2 -> 2 at 64 MiB 6.2 -> 6.9).
constexpr long kSmallBufferGroupPad = 20l << 10;
constexpr long kSmallBufferBytes = 96l << 20;

static std::mutex g_mem_mutex;
static std::unordered_map<void *, long> &mem_map() {
  static std::unordered_map<void *, long> m;
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
  const long gran = 2l << 20;
  const long rounded = (nbytes + gran - 1) / gran * gran;
  void *q = nullptr;
  hipError_t e = hipMalloc(&q, (size_t)rounded);
  if (e != hipSuccess || !q) {
    (void)hipGetLastError();
    return fail(PCCL_ERR_NOMEM, "hipMalloc(%ld): %s", rounded, hipGetErrorString(e));
  }
  std::lock_guard<std::mutex> lock(g_mem_mutex);
  mem_map()[q] = rounded;
  *p = q;
  return PCCL_OK;
}

int pccl_hip_alloc_group(void **ptrs, int n, long nbytes_each, long pad_bytes) {
  clear_error();
  if (!ptrs || n < 1) return fail(PCCL_ERR_INVALID_ARG, "pccl_hip_alloc_group: ptrs is null or n %d < 1", n);
  for (int k = 0; k < n; ++k) ptrs[k] = nullptr;
  if (nbytes_each <= 0) return fail(PCCL_ERR_INVALID_ARG, "pccl_hip_alloc_group: nbytes_each %ld <= 0", nbytes_each);
  if (pad_bytes < 0) pad_bytes = nbytes_each < kSmallBufferBytes ? kSmallBufferGroupPad : kDefaultGroupPad;
  pad_bytes = (pad_bytes + 255) / 256 * 256;
  const long stride = (nbytes_each + 255) / 256 * 256 + pad_bytes;
  const long gran = 2l << 20;
  const long rounded = ((long)n * stride + gran - 1) / gran * gran;
  void *q = nullptr;
  hipError_t e = hipMalloc(&q, (size_t)rounded);
  if (e != hipSuccess || !q) {
    (void)hipGetLastError();
    return fail(PCCL_ERR_NOMEM, "hipMalloc(%ld): %s", rounded, hipGetErrorString(e));
  }
  std::lock_guard<std::mutex> lock(g_mem_mutex);
  mem_map()[q] = rounded;  // the group is freed through its first buffer
  for (int k = 0; k < n; ++k) ptrs[k] = (char *)q + (long)k * stride;
  return PCCL_OK;
}

int pccl_hip_free(void *p) {
  clear_error();
  if (!p) return PCCL_OK;
  {
    std::lock_guard<std::mutex> lock(g_mem_mutex);
    auto it = mem_map().find(p);
    if (it == mem_map().end())
      return fail(PCCL_ERR_INVALID_ARG, "pccl_hip_free: %p was not allocated by pccl_hip_alloc", p);
    mem_map().erase(it);
  }
  PCCL_HIP_CHECK(hipFree(p));
  return PCCL_OK;
}

int pccl_hip_set_tuning(int workgroups_per_cu, int cache_treatment) {
  clear_error();
  if (workgroups_per_cu < 0 || workgroups_per_cu > 64)
    return fail(PCCL_ERR_INVALID_ARG, "workgroups_per_cu %d outside [0, 64]", workgroups_per_cu);
  (void)tuning();  // make sure the environment was read before overriding it
  std::lock_guard<std::mutex> lock(g_tuning_mutex);
  g_tuning.workgroups_per_cu = workgroups_per_cu;
  g_tuning.cache_treatment = cache_treatment < 0 ? -1 : std::min(cache_treatment, 2);
  return PCCL_OK;
}

int pccl_hip_set_unroll(int unroll) {
  clear_error();
  if (unroll != -1 && unroll != 0 && unroll != 1 && unroll != 4)
    return fail(PCCL_ERR_INVALID_ARG, "unroll %d is not -1, 0, 1 or 4", unroll);
  (void)tuning();
  std::lock_guard<std::mutex> lock(g_tuning_mutex);
  g_tuning.unroll = unroll;
  return PCCL_OK;
}

int pccl_hip_set_occupancy_lds(int lds_bytes) {
  clear_error();
  if (lds_bytes > 160 * 1024) return fail(PCCL_ERR_INVALID_ARG, "lds_bytes %d exceeds the 160 KiB of a compute unit", lds_bytes);
  (void)tuning();
  std::lock_guard<std::mutex> lock(g_tuning_mutex);
  g_tuning.lds_bytes = lds_bytes < 0 ? -1 : lds_bytes;
  return PCCL_OK;
}

const char *pccl_hip_last_error(void) { return g_error; }

int pccl_hip_dtype_bytes(int dtype) { return pccl_dtype_bytes(dtype); }

const char *pccl_hip_version(void) { return "pccl_hip 0.1 (gfx950)"; }

}  // extern "C"
