// reduce_copy_kernel.h -- the direct-launch reduce-copy kernel and its typed
// launcher.  One translation unit per dtype instantiates launch_typed<DT>, so
// the dtype x compute x n_in matrix compiles in parallel.
#pragma once

#include "plugin_common.h"
#include "reduce_copy_device.h"

namespace pccl_dev {

struct RcLaunch {
  RcOperands ops;  // original operand addresses
  long head;       // elements before the first 16-byte pack of output 0
  long n_packs;    // 16-byte packs in the body
  long count;      // elements in all
};

// Loads a lane keeps in flight per chunk: n_in * unroll packs of 16 bytes.
__host__ __device__ constexpr int unroll_for(int n_in) { return n_in >= 5 ? 1 : n_in >= 3 ? 2 : 8 / n_in; }

template <int DT, class Op, int NIN, bool ALIGNED, bool NT>
__global__ void __launch_bounds__(kBlock) reduce_copy_kernel(const RcLaunch p) {
  typedef Dtype<DT> D;
  constexpr int kEpp = 16 / D::kElemBytes;  // elements per pack
  if (p.n_packs > 0) {
    RcOperands body;
    body.n_out = p.ops.n_out;
#pragma unroll
    for (int k = 0; k < NIN; ++k) body.in[k] = p.ops.in[k] + p.head * D::kElemBytes;
#pragma unroll
    for (int j = 0; j < PCCL_MAX_OUTPUTS; ++j)
      if (j < p.ops.n_out) body.out[j] = p.ops.out[j] + p.head * D::kElemBytes;
    body_packs<D, Op, NIN, unroll_for(NIN), ALIGNED, NT>(body, p.n_packs, blockIdx.x, gridDim.x);
  }
  // head and tail elements: the last wavefront of the last workgroup
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x >= kBlock - kWave) {
    edge_elems<D, Op, NIN>(p.ops, p.head, p.head + p.n_packs * kEpp, p.count,
                           (int)threadIdx.x - (kBlock - kWave));
  }
}

template <int DT, class Op, int NIN>
int launch_nin(bool aligned, bool nt, unsigned grid, hipStream_t stream, const RcLaunch &p) {
  if (aligned) {
    if (nt) hipLaunchKernelGGL((reduce_copy_kernel<DT, Op, NIN, true, true>), dim3(grid), dim3(kBlock), 0, stream, p);
    else hipLaunchKernelGGL((reduce_copy_kernel<DT, Op, NIN, true, false>), dim3(grid), dim3(kBlock), 0, stream, p);
  } else {
    if (nt) hipLaunchKernelGGL((reduce_copy_kernel<DT, Op, NIN, false, true>), dim3(grid), dim3(kBlock), 0, stream, p);
    else hipLaunchKernelGGL((reduce_copy_kernel<DT, Op, NIN, false, false>), dim3(grid), dim3(kBlock), 0, stream, p);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return pccl_host::fail(PCCL_ERR_HIP, "reduce_copy launch failed: %s", hipGetErrorString(e));
  return PCCL_OK;
}

template <int DT, class Op>
int launch_op(int n_in, bool aligned, bool nt, unsigned grid, hipStream_t stream, const RcLaunch &p) {
  switch (n_in) {
    case 2: return launch_nin<DT, Op, 2>(aligned, nt, grid, stream, p);
    case 3: return launch_nin<DT, Op, 3>(aligned, nt, grid, stream, p);
    case 4: return launch_nin<DT, Op, 4>(aligned, nt, grid, stream, p);
    case 5: return launch_nin<DT, Op, 5>(aligned, nt, grid, stream, p);
    case 6: return launch_nin<DT, Op, 6>(aligned, nt, grid, stream, p);
    case 7: return launch_nin<DT, Op, 7>(aligned, nt, grid, stream, p);
    case 8: return launch_nin<DT, Op, 8>(aligned, nt, grid, stream, p);
    default: return pccl_host::fail(PCCL_ERR_INVALID_ARG, "n_in %d outside [1, 8]", n_in);
  }
}

// n_in >= 2.  Defined once per dtype (reduce_copy_inst_*.hip).
template <int DT>
int launch_typed(int compute, int n_in, bool aligned, bool nt, unsigned grid, hipStream_t stream,
                 const RcLaunch &p);

// n_in == 1: bytes move unchanged, so only the element size matters.
int launch_copy(int elem_bytes, bool aligned, bool nt, unsigned grid, hipStream_t stream,
                const RcLaunch &p);

#define PCCL_DEFINE_LAUNCH_TYPED(DT)                                                            \
  template <>                                                                                   \
  int launch_typed<DT>(int compute, int n_in, bool aligned, bool nt, unsigned grid,             \
                       hipStream_t stream, const RcLaunch &p) {                                 \
    switch (compute) {                                                                          \
      case PCCL_SUM: return launch_op<DT, OpSum>(n_in, aligned, nt, grid, stream, p);           \
      case PCCL_PROD: return launch_op<DT, OpProd>(n_in, aligned, nt, grid, stream, p);         \
      case PCCL_MIN: return launch_op<DT, OpMin>(n_in, aligned, nt, grid, stream, p);           \
      case PCCL_MAX: return launch_op<DT, OpMax>(n_in, aligned, nt, grid, stream, p);           \
      default: return pccl_host::fail(PCCL_ERR_UNSUPPORTED, "unknown compute code %d", compute); \
    }                                                                                           \
  }

}  // namespace pccl_dev
