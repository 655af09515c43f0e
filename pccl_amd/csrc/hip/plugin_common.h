// plugin_common.h -- host-side helpers shared by the translation units of
// libpccl_hip.so: thread-local error text and HIP call checking.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "pccl_hip.h"

namespace pccl_host {

// Sets the calling thread's error text and returns `code` so that call sites
// can write `return fail(PCCL_ERR_..., "...")`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

inline int pccl_dtype_bytes(int dtype) {
  return dtype == PCCL_F64 ? 8 : dtype == PCCL_F32 || dtype == PCCL_I32 || dtype == PCCL_U32 ? 4
         : dtype == PCCL_BF16 || dtype == PCCL_F16 ? 2 : dtype == PCCL_F8E4M3 || dtype == PCCL_F8E5M2 ? 1 : 0;
}

// Compute units of the current device (cached per device index).
int compute_units();

// What pccl_hip_set_executor_id was given (0 before any call).
int executor_id();

struct Tuning {
  int workgroups_per_cu;  // 0 = built-in choice
  int cache_treatment;        // -1 = built-in choice, else 0 cacheable / 1 streaming / 2 streaming loads + write-through stores
  int lds_bytes;          // -1 = built-in choice, else dynamic LDS requested per workgroup
  int unroll;             // -1 = built-in choice, 0 = lean kernel where it applies, else packs per lane (1 or 4)
  int rotate;             // -1 = built-in choice, 0 = workgroup k takes chunk k, 1 = rotated wherever the launch shape allows
};
Tuning tuning();

// Longest stretch of an operand, in bytes, that one launch of pccl_hip_reduce_copy / pccl_hip_accumulate
// covers (a multiple of 4 KiB; see pccl_hip_set_slice_bytes).
long slice_bytes();

}  // namespace pccl_host

#define PCCL_HIP_CHECK(expr)                                                              \
  do {                                                                                    \
    hipError_t _e = (expr);                                                               \
    if (_e != hipSuccess)                                                                 \
      return ::pccl_host::fail(PCCL_ERR_HIP, "%s failed: %s (%s:%d)", #expr,              \
                               hipGetErrorString(_e), __FILE__, __LINE__);                \
  } while (0)
