// accumulate.hip -- pccl_hip_accumulate: fold ONE input into each of K destinations,
//   outs[j][i] = cvt(op(up(outs[j][i]), up(in[i]))),
// reading the input once.  Fills the role of multimemStoreReduce (reference
// include/plugins/cuda_executor/utils/multimem.h:104-127: multimem.red.add of one
// register pack into every peer's copy; only .add and only f32 / f16x2 there).
// The destination is the accumulator (input 0 of the fold), the value is input 1;
// each destination element is read and written by the same lane, so no atomics
// are needed as long as nobody else writes the destinations during the launch.
#include <algorithm>
#include <cstring>

#include "plugin_common.h"
#include "reduce_copy_kernel.h"

using namespace pccl_dev;
using pccl_host::fail;

namespace {

struct AccLaunch {
  const char *in;
  char *out[PCCL_MAX_OUTPUTS];
  int n_out;
  long head;     // elements before the first 16-byte pack of output 0
  long n_packs;  // 16-byte packs in the body
  long count;
  int rotate;    // workgroup -> chunk rotation (rotated_chunk, reduce_copy_kernel.h)
};

// One pack per lane with a compile-time number of destinations: 1 + NOUT loads in flight per
// lane, then the folds and stores (the destinations are distinct buffers by contract, so
// nothing written here is read here).  With the count a run-time bound on loops over an array
// of packs the compiler carried the whole array through every branch for f32 and f64 (240
// VGPRs, two wavefronts per SIMD: f32 1 -> 7 at 4.6 TB/s where bf16 reached 6.35).
// How the stores leave matters once the streams are many, and differently for few and for many
// destinations (128 MiB operands, medians over fresh allocations, all dtypes):
//   3-4 destinations: every fold first, then the stores in one burst   6.4-6.5 TB/s
//                     (folds and stores interleaved: 5.9-6.4, by the fold's length)
//   5-8 destinations: fold and store one destination after the other, with a pause of 128
//                     clocks (8 destinations: 320; 5-6 destinations of a 1- or 2-byte type,
//                     whose folds are long: 64) between the stores      6.2-6.5 TB/s
//                     (no pause: 5.6-5.7 for the short folds of i32 / f32 / f64, 6.1-6.5 for
//                     the longer ones of bf16 / f16 / f8, whose arithmetic paces them anyway;
//                     one burst: 5.5-5.8)
template <class D, class Op, bool ALIGNED, int LD, int ST, int NOUT>
__device__ __forceinline__ void accumulate_pack(const AccLaunch &p, size_t wg, unsigned int off) {
  const u32x4 x = load_pack<D, ALIGNED, LD>(p.in + wg, off);
  u32x4 d[NOUT];
#pragma unroll
  for (int j = 0; j < NOUT; ++j)  // output 0 is 16-byte aligned by the peel; the others only if ALIGNED
    d[j] = j == 0 ? load_pack<D, true, LD>(p.out[0] + wg, off) : load_pack<D, ALIGNED, LD>(p.out[j] + wg, off);
  if constexpr (NOUT <= 2) {
#pragma unroll
    for (int j = 0; j < NOUT; ++j) {
      const u32x4 v[2] = {d[j], x};
      const u32x4 r = fold_pack<D, Op, 2>(v);
      if (j == 0) store_pack<D, true, ST>(p.out[0] + wg, off, r);
      else store_pack<D, ALIGNED, ST>(p.out[j] + wg, off, r);
    }
  } else if constexpr (NOUT <= 4) {
    // every load back, every fold done, then the stores in one burst
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < NOUT; ++j) {
      const u32x4 v[2] = {d[j], x};
      d[j] = fold_pack<D, Op, 2>(v);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < NOUT; ++j) {
      if (j == 0) store_pack<D, true, ST>(p.out[0] + wg, off, d[0]);
      else store_pack<D, ALIGNED, ST>(p.out[j] + wg, off, d[j]);
    }
  } else {
    // every load back, then fold and store destination after destination, the stores spaced
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int j = 0; j < NOUT; ++j) {
      const u32x4 v[2] = {d[j], x};
      const u32x4 r = fold_pack<D, Op, 2>(v);
      if (j == 0) store_pack<D, true, ST>(p.out[0] + wg, off, r);
      else store_pack<D, ALIGNED, ST>(p.out[j] + wg, off, r);
      if (j + 1 < NOUT) __builtin_amdgcn_s_sleep(NOUT == 8 ? 5 : (D::kElemBytes < 4 && NOUT <= 6) ? 1 : 2);
    }
  }
}

// ALIGNED: input and every output 16-byte aligned after the head peel.
// MEM: cache treatment as for reduce_copy (0 cacheable, 1 streaming, 2 streaming loads and
// write-through stores).
template <int DT, class Op, bool ALIGNED, int MEM>
__global__ void __launch_bounds__(kBlock) accumulate_kernel(const AccLaunch p) {
  constexpr int kLd = LaunchMem<MEM, 2>::kLd, kSt = LaunchMem<MEM, 2>::kSt;
  typedef Dtype<DT> D;
  D::wave_init();
  typedef typename D::elem_t E;
  constexpr int kEpp = 16 / D::kElemBytes;
  const unsigned chunk = p.rotate ? rotated_chunk(blockIdx.x, gridDim.x) : blockIdx.x;
  const long pack = (long)chunk * kBlock + threadIdx.x;
  if (pack < p.n_packs) {
    // (wave-uniform base, lane offset) addressing: the workgroup's 4 KiB of every stream
    const size_t wg = (size_t)p.head * D::kElemBytes + (size_t)chunk * (kBlock * 16);
    const unsigned int off = threadIdx.x * 16u;
    switch (p.n_out) {
      case 1: accumulate_pack<D, Op, ALIGNED, kLd, kSt, 1>(p, wg, off); break;
      case 2: accumulate_pack<D, Op, ALIGNED, kLd, kSt, 2>(p, wg, off); break;
      case 3: accumulate_pack<D, Op, ALIGNED, kLd, kSt, 3>(p, wg, off); break;
      case 4: accumulate_pack<D, Op, ALIGNED, kLd, kSt, 4>(p, wg, off); break;
      case 5: accumulate_pack<D, Op, ALIGNED, kLd, kSt, 5>(p, wg, off); break;
      case 6: accumulate_pack<D, Op, ALIGNED, kLd, kSt, 6>(p, wg, off); break;
      case 7: accumulate_pack<D, Op, ALIGNED, kLd, kSt, 7>(p, wg, off); break;
      default: accumulate_pack<D, Op, ALIGNED, kLd, kSt, 8>(p, wg, off); break;
    }
  }
  // head and tail elements: the last wavefront of the last workgroup
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x >= kBlock - kWave) {
    const long tail_begin = p.head + p.n_packs * kEpp;
    const long n_edge = p.head + (p.count - tail_begin);
    for (long e = (long)threadIdx.x - (kBlock - kWave); e < n_edge; e += kWave) {
      const long i = e < p.head ? e : tail_begin + (e - p.head);
      E x[2];
      x[1] = ((const E *)p.in)[i];
#pragma unroll
      for (int j = 0; j < PCCL_MAX_OUTPUTS; ++j)
        if (j < p.n_out) {
          x[0] = ((const E *)p.out[j])[i];
          ((E *)p.out[j])[i] = D::template elem<Op, 2>(x);
        }
    }
  }
}

template <int DT, class Op>
int launch_acc(bool aligned, int mem, unsigned grid, unsigned lds, hipStream_t stream, const AccLaunch &p) {
  with_launch_mem(mem, [&](auto m) {
    constexpr int kMem = decltype(m)::value;
    if (aligned) hipLaunchKernelGGL((accumulate_kernel<DT, Op, true, kMem>), dim3(grid), dim3(kBlock), lds, stream, p);
    else hipLaunchKernelGGL((accumulate_kernel<DT, Op, false, kMem>), dim3(grid), dim3(kBlock), lds, stream, p);
  });
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(PCCL_ERR_HIP, "accumulate launch failed: %s", hipGetErrorString(e));
  return PCCL_OK;
}

template <int DT>
int launch_acc_op(int compute, bool aligned, int mem, unsigned grid, unsigned lds, hipStream_t stream,
                  const AccLaunch &p) {
  switch (compute) {
    case PCCL_SUM: return launch_acc<DT, OpSum>(aligned, mem, grid, lds, stream, p);
    case PCCL_PROD: return launch_acc<DT, OpProd>(aligned, mem, grid, lds, stream, p);
    case PCCL_MIN: return launch_acc<DT, OpMin>(aligned, mem, grid, lds, stream, p);
    default: return launch_acc<DT, OpMax>(aligned, mem, grid, lds, stream, p);
  }
}

}  // namespace

extern "C" int pccl_hip_accumulate(int dtype, int compute, const void *in, void *const *outs, int n_out,
                                   long count, void *stream) {
  pccl_host::clear_error();
  if (dtype < 0 || dtype >= PCCL_NUM_DTYPES) return fail(PCCL_ERR_UNSUPPORTED, "unknown dtype code %d", dtype);
  if (compute < PCCL_SUM || compute > PCCL_MAX) return fail(PCCL_ERR_UNSUPPORTED, "unknown compute code %d", compute);
  if (n_out < 1 || n_out > PCCL_MAX_OUTPUTS) return fail(PCCL_ERR_INVALID_ARG, "n_out %d outside [1, 8]", n_out);
  if (count < 0) return fail(PCCL_ERR_INVALID_ARG, "count %ld < 0", count);
  if (!outs) return fail(PCCL_ERR_INVALID_ARG, "output array is null");
  const int es = pccl_host::pccl_dtype_bytes(dtype);
  if (!in && count) return fail(PCCL_ERR_INVALID_ARG, "input is null");
  if ((uintptr_t)in % es) return fail(PCCL_ERR_MISALIGNED, "input (%p) not %d-byte aligned", in, es);
  AccLaunch p;
  memset(&p, 0, sizeof(p));
  p.in = (const char *)in;
  for (int j = 0; j < n_out; ++j) {
    if (!outs[j] && count) return fail(PCCL_ERR_INVALID_ARG, "output %d is null", j);
    if ((uintptr_t)outs[j] % es) return fail(PCCL_ERR_MISALIGNED, "output %d (%p) not %d-byte aligned", j, outs[j], es);
    for (int k = 0; k < j; ++k)
      if (outs[k] == outs[j]) return fail(PCCL_ERR_INVALID_ARG, "outputs %d and %d are the same buffer", k, j);
    p.out[j] = (char *)outs[j];
  }
  if (count == 0) return PCCL_OK;
  // (one workgroup per 4 KiB of every stream, and a grid times its 256 lanes must fit 32 bits: operands
  // beyond 32 GiB run as launches over consecutive slices of that size, like pccl_hip_reduce_copy's)
  const long slice = pccl_host::slice_bytes() / es;
  if (count > slice) {
    for (long lo = 0; lo < count; lo += slice) {
      void *out_at[PCCL_MAX_OUTPUTS];
      for (int j = 0; j < n_out; ++j) out_at[j] = (char *)outs[j] + lo * es;
      const int rc = pccl_hip_accumulate(dtype, compute, (const char *)in + lo * es, out_at, n_out, std::min(slice, count - lo), stream);
      if (rc != PCCL_OK) return rc;
    }
    return PCCL_OK;
  }
  p.n_out = n_out;
  p.count = count;
  p.head = std::min<long>(count, (long)((16 - ((uintptr_t)outs[0] & 15)) & 15) / es);
  p.n_packs = (count - p.head) / (16 / es);
  bool aligned = (((uintptr_t)in + (uintptr_t)p.head * es) & 15) == 0;
  for (int j = 0; j < n_out; ++j) aligned = aligned && (((uintptr_t)outs[j] + (uintptr_t)p.head * es) & 15) == 0;
  const unsigned grid = (unsigned)std::max<long>(1, (p.n_packs + kBlock - 1) / kBlock);
  // Launch policy, measured on MI355X (128 MiB operands unless noted).  A lane has 1 + n_out
  // loads in flight, then n_out stores.  Cache treatment: one destination, or input and
  // destinations fitting the 256 MB Infinity Cache together, prefer cached accesses (1 -> 1:
  // 7.3 vs 6.5 TB/s; 1 -> 7 at 32 MiB: 6.8 vs 5.7); two destinations streaming loads with
  // write-through stores (7.1 vs 5.9 non-temporal, 5.6 cached); three and more non-temporal
  // loads and stores (1 -> 7: 6.3 vs 6.0 cached or write-through).  Beyond the cache the
  // occupancy cap of reduce_copy applies with 1 + 2 n_out streams per workgroup: about 20
  // (workgroups x streams) per compute unit, at least 2 workgroups (1 -> 7: 6.3 with 2 or 3
  // workgroups resident, 5.6-5.8 with 4 and more; 1 -> 3: 6.25 with 3, 5.9-6.0 otherwise).
  const pccl_host::Tuning t = pccl_host::tuning();
  const long total_bytes = (long)(1 + 2 * n_out) * count * es;
  const long working_set = (long)(1 + n_out) * count * es;
  const bool beyond_cache = total_bytes > (192l << 20) && (n_out <= 2 || working_set > (256l << 20));
  int mem = kLaunchMemCached;
  if (n_out == 2 && total_bytes >= (48l << 20))
    mem = total_bytes > (192l << 20) ? kLaunchMemStreamWriteThrough : kLaunchMemStream;
  else if (n_out >= 3 && working_set > (256l << 20)) mem = kLaunchMemStream;
  if (t.cache_treatment >= 0) mem = std::min(t.cache_treatment, (int)kLaunchMemStreamWriteThrough);
  unsigned lds = 0;
  if (t.lds_bytes >= 0) {
    lds = (unsigned)t.lds_bytes;
  } else if (beyond_cache) {
    const int streams = 1 + 2 * n_out;
    const int wgs = std::max(2, std::min(8, (20 + streams / 2) / streams));
    if (wgs < 8) lds = std::min(65536u, (unsigned)(160 * 1024 / wgs) - 256u);
  }
  // the chunk order of large launches, as for reduce_copy (one workgroup per chunk here always)
  // (and, as there, not for operands of 4 GiB and more each)
  p.rotate = t.rotate > 0 || (t.rotate != 0 && beyond_cache && count * es < (4l << 30));
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case PCCL_F32: return launch_acc_op<PCCL_F32>(compute, aligned, mem, grid, lds, s, p);
    case PCCL_I32: return launch_acc_op<PCCL_I32>(compute, aligned, mem, grid, lds, s, p);
    case PCCL_BF16: return launch_acc_op<PCCL_BF16>(compute, aligned, mem, grid, lds, s, p);
    case PCCL_F16: return launch_acc_op<PCCL_F16>(compute, aligned, mem, grid, lds, s, p);
    case PCCL_F8E4M3: return launch_acc_op<PCCL_F8E4M3>(compute, aligned, mem, grid, lds, s, p);
    case PCCL_F8E5M2: return launch_acc_op<PCCL_F8E5M2>(compute, aligned, mem, grid, lds, s, p);
    case PCCL_F64: return launch_acc_op<PCCL_F64>(compute, aligned, mem, grid, lds, s, p);
    default: return launch_acc_op<PCCL_U32>(compute, aligned, mem, grid, lds, s, p);
  }
}
