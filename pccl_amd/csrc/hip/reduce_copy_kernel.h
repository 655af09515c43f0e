// reduce_copy_kernel.h -- the direct-launch reduce-copy kernel and its typed
// launcher.  One translation unit per dtype instantiates launch_typed<DT>, so
// the dtype x compute x n_in matrix compiles in parallel.
#pragma once

#include <type_traits>

#include "plugin_common.h"
#include "reduce_copy_device.h"

namespace pccl_dev {

struct RcLaunch {
  RcOperands ops;  // original operand addresses
  long head;       // elements before the first 16-byte pack of output 0
  long n_packs;    // 16-byte packs in the body
  long count;      // elements in all
  int rotate;      // workgroup -> chunk rotation (rotated_chunk below); needs grid == number of chunks
};

// Which 4 KiB chunk of every stream workgroup k works on.  The hardware hands workgroups to the 8 XCDs
// in turn (workgroup k runs on XCD k % 8), and address bits 12-14 of a chunk select, together with
// higher bits, one of the 8 groups of 16 HBM channels.  With chunk = k every XCD reads each stream
// from ONE group for the whole launch, and when the streams' addresses agree in the group bits (buffers
// a power of two apart do, in all but one of them) from one or two groups in all: one XCD-to-group
// path then carries an eighth of the traffic and tops out near 650 GB/s (8 lockstep read streams in
// one group: 5.2 TB/s).  XORing bits 5-7 of k into its low three bits sends the 4 consecutive
// workgroups an XCD gets out of every 32 to the same group (4 x 256 bytes = one 1 KiB DRAM page
// per channel stays together) and the next 4 to another, so that the workgroups in flight on an XCD
// cover all 8 groups whatever the addresses are.  bf16 8 -> 1, TB/s without -> with, by how far the
// nine buffers are apart: their size (nine separate allocations) 256 MiB 6.56 -> 6.95, 128 MiB
// 6.63 -> 7.11; size + 8 KiB 5.23 -> 6.87; size + 2 MiB 4.90 -> 6.98; 1 GiB 4.88 -> 7.01; size + 4 KiB
// (the best case without) 6.90 -> 6.67.  Rotating every 8 workgroups loses the DRAM pages (6.3),
// every 64 recovers less (6.1-6.9), every 256 nothing.  Cache-resident sizes do not gain (copies of
// 32-64 MiB lose 5 %), so the launch asks for it only beyond the Infinity Cache.
__device__ __forceinline__ unsigned rotated_chunk(unsigned k, unsigned n_chunks) {
  // a permutation inside every aligned run of 8 chunks; the last, partial run keeps its order
  return (k | 7u) < n_chunks ? k ^ ((k >> 5) & 7u) : k;
}

// Packs per lane per workgroup.  Measured on MI355X: with streams larger than
// the Infinity Cache one pack per lane and one workgroup per 4 KiB of every stream
// (the hardware dispatcher then walks memory in address order) beats every
// persistent / grid-stride shape for all n_in; only cache-resident copies and
// 2-input reductions gain (about 5 %) from 4 packs per lane in this, the general kernel
// (the lean kernel, taken wherever it applies, has one pack per lane throughout).
__host__ __device__ constexpr int small_unroll_for(int n_in) { return n_in <= 2 ? 4 : 1; }

// MEM: how the launch treats the caches (host-side choice by operand size and shape).
//   0  everything cacheable;
//   1  streaming: non-temporal loads and stores (a copy: stores only);
//   2  non-temporal loads (a copy too), write-through (sc1) stores.  Measured on MI355X this
//      beats 1 for reductions beyond the caches (bf16 8 -> 2 at 128 MiB 6.5 -> 6.9 TB/s,
//      2 -> 1 at 256 MiB 6.6 -> 7.2) and for the steps of a ring walk, copies included.
constexpr int kLaunchMemCached = 0, kLaunchMemStream = 1, kLaunchMemStreamWriteThrough = 2;
template <int MEM, int NIN> struct LaunchMem {
  static constexpr int kLd =
      (MEM == kLaunchMemStreamWriteThrough || (MEM == kLaunchMemStream && NIN > 1)) ? kMemStream : kMemCached;
  static constexpr int kSt = MEM == kLaunchMemCached ? kMemCached : MEM == kLaunchMemStream ? kMemStream : kMemCoherent;
};

// Calls f(std::integral_constant<int, mem>) for mem in 0..2.
template <class F>
inline void with_launch_mem(int mem, F &&f) {
  if (mem == kLaunchMemStreamWriteThrough) f(std::integral_constant<int, kLaunchMemStreamWriteThrough>{});
  else if (mem == kLaunchMemStream) f(std::integral_constant<int, kLaunchMemStream>{});
  else f(std::integral_constant<int, kLaunchMemCached>{});
}

template <int DT, class Op, int NIN, int UNROLL, bool ALIGNED, int MEM>
__global__ void __launch_bounds__(kBlock) reduce_copy_kernel(const RcLaunch p) {
  typedef Dtype<DT> D;
  if constexpr (NIN > 1) D::wave_init();
  constexpr int kEpp = 16 / D::kElemBytes;  // elements per pack
  if (p.n_packs > 0) {
    RcOperands body;
    body.n_out = p.ops.n_out;
#pragma unroll
    for (int k = 0; k < NIN; ++k) body.in[k] = p.ops.in[k] + p.head * D::kElemBytes;
#pragma unroll
    for (int j = 0; j < PCCL_MAX_OUTPUTS; ++j)
      if (j < p.ops.n_out) body.out[j] = p.ops.out[j] + p.head * D::kElemBytes;
    // (UNROLL == 1 whenever rotate is set: a chunk is then 4 KiB and the grid has one workgroup per chunk)
    const unsigned wg = p.rotate ? rotated_chunk(blockIdx.x, gridDim.x) : blockIdx.x;
    body_packs<D, Op, NIN, UNROLL, ALIGNED, LaunchMem<MEM, NIN>::kLd, LaunchMem<MEM, NIN>::kSt>(
        body, p.n_packs, wg, gridDim.x);
  }
  // head and tail elements: the last wavefront of the last workgroup
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x >= kBlock - kWave) {
    edge_elems<D, Op, NIN>(p.ops, p.head, p.head + p.n_packs * kEpp, p.count,
                           (int)threadIdx.x - (kBlock - kWave));
  }
}

// ---- lean kernel for the common case -------------------------------------------
// Every stream 16-byte aligned, count a whole number of packs, at most two
// outputs: one pack per lane, one workgroup per 4 KiB of every stream, no loop,
// no edge code.  A workgroup lives for only a few microseconds, so what it does
// before its first load matters: the arguments hold nothing but the pointers it
// needs, the per-workgroup offset is added on the scalar unit and the per-lane
// offset is a 32-bit value (scalar-base addressing, no 64-bit vector adds).
template <int NIN, int NOUT>
struct RcLean {
  const char *in[NIN];
  char *out[NOUT];
  long n_packs;
  int rotate;
};

template <int DT, class Op, int NIN, int NOUT, int MEM>
__global__ void __launch_bounds__(kBlock) reduce_copy_lean_kernel(const RcLean<NIN, NOUT> a) {
  typedef Dtype<DT> D;
  if constexpr (NIN > 1) D::wave_init();
  constexpr int kLd = LaunchMem<MEM, NIN>::kLd;
  constexpr int kSt = LaunchMem<MEM, NIN>::kSt;
  const unsigned lane_off = threadIdx.x * 16u;
  const unsigned chunk = a.rotate ? rotated_chunk(blockIdx.x, gridDim.x) : blockIdx.x;
  const size_t wg_off = (size_t)chunk * (kBlock * 16);
  if ((long)chunk * kBlock + threadIdx.x < a.n_packs) {
    u32x4 v[NIN];
#pragma unroll
    for (int k = 0; k < NIN; ++k) v[k] = load_pack<D, true, kLd>(a.in[k] + wg_off, lane_off);
    const u32x4 r = fold_pack<D, Op, NIN>(v);
#pragma unroll
    for (int j = 0; j < NOUT; ++j) store_pack<D, true, kSt>(a.out[j] + wg_off, lane_off, r);
  }
}

template <int DT, class Op, int NIN, int NOUT>
int launch_lean_nout(int mem, unsigned lds, hipStream_t stream, const RcLaunch &p) {
  RcLean<NIN, NOUT> a;
  for (int k = 0; k < NIN; ++k) a.in[k] = p.ops.in[k];
  for (int j = 0; j < NOUT; ++j) a.out[j] = p.ops.out[j];
  a.n_packs = p.n_packs;
  a.rotate = p.rotate;
  const unsigned grid = (unsigned)((p.n_packs + kBlock - 1) / kBlock);
  with_launch_mem(mem, [&](auto m) {
    hipLaunchKernelGGL((reduce_copy_lean_kernel<DT, Op, NIN, NOUT, decltype(m)::value>), dim3(grid), dim3(kBlock), lds, stream, a);
  });
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return pccl_host::fail(PCCL_ERR_HIP, "reduce_copy launch failed: %s", hipGetErrorString(e));
  return PCCL_OK;
}

// requires: p.head == 0, p.n_packs * pack == p.count, all streams aligned, n_out <= 2
template <int DT, class Op, int NIN>
int launch_lean(int mem, unsigned lds, hipStream_t stream, const RcLaunch &p) {
  if (p.ops.n_out == 1) return launch_lean_nout<DT, Op, NIN, 1>(mem, lds, stream, p);
  return launch_lean_nout<DT, Op, NIN, 2>(mem, lds, stream, p);
}

template <int DT, class Op, int NIN, int UNROLL>
int launch_shape(bool aligned, int mem, unsigned grid, unsigned lds, hipStream_t stream, const RcLaunch &p) {
  with_launch_mem(mem, [&](auto m) {
    constexpr int kMem = decltype(m)::value;
    if (aligned) hipLaunchKernelGGL((reduce_copy_kernel<DT, Op, NIN, UNROLL, true, kMem>), dim3(grid), dim3(kBlock), lds, stream, p);
    else hipLaunchKernelGGL((reduce_copy_kernel<DT, Op, NIN, UNROLL, false, kMem>), dim3(grid), dim3(kBlock), lds, stream, p);
  });
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return pccl_host::fail(PCCL_ERR_HIP, "reduce_copy launch failed: %s", hipGetErrorString(e));
  return PCCL_OK;
}

// unroll is 0 (lean kernel), 1 or small_unroll_for(NIN); the last two coincide for n_in >= 3
template <int DT, class Op, int NIN>
int launch_nin(int unroll, bool aligned, int mem, unsigned grid, unsigned lds, hipStream_t stream, const RcLaunch &p) {
  if (unroll == 0) return launch_lean<DT, Op, NIN>(mem, lds, stream, p);
  if constexpr (small_unroll_for(NIN) != 1) {
    if (unroll != 1) return launch_shape<DT, Op, NIN, small_unroll_for(NIN)>(aligned, mem, grid, lds, stream, p);
  }
  return launch_shape<DT, Op, NIN, 1>(aligned, mem, grid, lds, stream, p);
}

template <int DT, class Op>
int launch_op(int n_in, int unroll, bool aligned, int mem, unsigned grid, unsigned lds, hipStream_t stream,
              const RcLaunch &p) {
  switch (n_in) {
    case 2: return launch_nin<DT, Op, 2>(unroll, aligned, mem, grid, lds, stream, p);
    case 3: return launch_nin<DT, Op, 3>(unroll, aligned, mem, grid, lds, stream, p);
    case 4: return launch_nin<DT, Op, 4>(unroll, aligned, mem, grid, lds, stream, p);
    case 5: return launch_nin<DT, Op, 5>(unroll, aligned, mem, grid, lds, stream, p);
    case 6: return launch_nin<DT, Op, 6>(unroll, aligned, mem, grid, lds, stream, p);
    case 7: return launch_nin<DT, Op, 7>(unroll, aligned, mem, grid, lds, stream, p);
    case 8: return launch_nin<DT, Op, 8>(unroll, aligned, mem, grid, lds, stream, p);
    default: return pccl_host::fail(PCCL_ERR_INVALID_ARG, "n_in %d outside [1, 8]", n_in);
  }
}

// n_in >= 2.  Defined once per dtype (reduce_copy_inst_*.hip).
template <int DT>
int launch_typed(int compute, int n_in, int unroll, bool aligned, int mem, unsigned grid, unsigned lds,
                 hipStream_t stream, const RcLaunch &p);

// n_in == 1: bytes move unchanged, so only the element size matters.
int launch_copy(int elem_bytes, int unroll, bool aligned, int mem, unsigned grid, unsigned lds,
                hipStream_t stream, const RcLaunch &p);

#define PCCL_DEFINE_LAUNCH_TYPED(DT)                                                            \
  template <>                                                                                   \
  int launch_typed<DT>(int compute, int n_in, int unroll, bool aligned, int mem, unsigned grid, \
                       unsigned lds, hipStream_t stream, const RcLaunch &p) {                   \
    switch (compute) {                                                                          \
      case PCCL_SUM: return launch_op<DT, OpSum>(n_in, unroll, aligned, mem, grid, lds, stream, p);           \
      case PCCL_PROD: return launch_op<DT, OpProd>(n_in, unroll, aligned, mem, grid, lds, stream, p);         \
      case PCCL_MIN: return launch_op<DT, OpMin>(n_in, unroll, aligned, mem, grid, lds, stream, p);           \
      case PCCL_MAX: return launch_op<DT, OpMax>(n_in, unroll, aligned, mem, grid, lds, stream, p);           \
      default: return pccl_host::fail(PCCL_ERR_UNSUPPORTED, "unknown compute code %d", compute); \
    }                                                                                           \
  }

}  // namespace pccl_dev
