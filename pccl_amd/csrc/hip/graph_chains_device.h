// graph_chains_device.h -- a graph of independent chains as ONE launch in the shape of the direct
// kernels: the chains' operands come through a table that all workgroups share.
//
// Open to graphs whose queue entries wait for nothing (as for any wide launch, graph_queue_device.h)
// when every entry is either one op or a chain that comes down to "fold these inputs, store the
// result to these outputs": the head's inputs folded like one reduction, then one more input per
// later op, each fold rounded to the element type where the op's store would round it, and every
// output that survives (an output that a later op of the chain writes again is never stored) holding
// the chain's final value.  A ring all-reduce over ranks that live on one device is eight such
// chains (eight inputs, eight outputs each), a direct all-reduce eight folds 8 -> 8.
// A workgroup takes 4 KiB of every stream of its chain, one pack per lane: all loads at once, the
// folds, all stores, like reduce_copy_lean_kernel (packs cut on output 0's 16-byte boundaries, the other
// operands at whatever element-aligned address that gives them, the few elements in front of the
// first and behind the last pack by the chain's last workgroup).  Which chain a workgroup belongs to
// follows from the launch's arguments alone (first workgroup of every chain; with more than
// kLaunchChainGroups chains, of every group of chains, and the rows of the group say the rest); the chain's row of the table is the same
// for all its workgroups, so it is fetched once per compute unit and then comes from the scalar cache:
// no per-entry record, no table staged through LDS, no barrier in front of the first load, and
// workgroups that live a fifth as long as a wide launch's 16 KiB entries, which is what that launch
// loses against a direct one at both ends of an entry's life.  Ring all-reduce over 8 resident ranks,
// 112 ops, wide launch -> this: see graph_queue.hip (launch_chains_of).
// The table lives in the graph's arena: a rebind rewrites it like the payloads, and launches that a
// stream capture has recorded follow.
#pragma once
#include "graph_queue_device.h"
#include "reduce_copy_kernel.h"

namespace pccl_queue {

constexpr int kLaunchChainGroups = 16;  // chains, or groups of up to kLaunchChainsPerGroup chains, that the launch's arguments name
constexpr int kLaunchChainsPerGroup = 4;
constexpr int kMaxLaunchChains = kLaunchChainGroups * kLaunchChainsPerGroup;
constexpr int kChainStreams = 8;  // inputs, and outputs, of one chain

struct LaunchChain {
  unsigned long long in[kChainStreams];   // the head's inputs, then the other input of every later op that has one
  unsigned long long out[kChainStreams];  // the surviving outputs
  long long count;                        // elements of every stream
  int n_head;                             // inputs folded as one reduction (the head op's)
  int n_in, n_out;
  unsigned int fed;                       // bit k (k >= n_head): the handed-on value is the second operand of the fold with input k
  int uid;                                // the head op (trace records)
  unsigned int n_wg;                      // workgroups of this chain: one per 4 KiB of floor(bytes / 16) packs, at least one
  unsigned int first_wg;                  // the chain's first workgroup
  int reserved[7];
};
static_assert(sizeof(LaunchChain) == 192, "launch chain row");

// The launch's arguments.  Nothing here depends on an address (a recorded launch keeps its copy).
struct ChainsLaunch {
  const LaunchChain *chains;
  unsigned long long *trace;                 // per workgroup: kTraceWords words, or null
  unsigned int first_wg[kLaunchChainGroups];  // first workgroup of chain k * group; beyond the last chain: 0xffffffff
  int rotate;                                 // workgroup -> chunk rotation inside a chain (rotated_chunk)
  int group;                                  // 1 for up to kLaunchChainGroups chains (the arguments alone say which chain a
                                              // workgroup belongs to: a launch of many short-lived workgroups loses 5-8 % to
                                              // a longer argument block), else up to kLaunchChainsPerGroup: the rows' first_wg decide
  int n_chains;
};

// One workgroup's 4 KiB of a chain of NIN inputs (a count the compiler knows: a register array that is
// written under run-time conditions costs the floating-point instances 244 registers and a wait behind
// every load).  n_head is NIN (one op: all inputs folded as one reduction) or, for a one-pass chain, the
// head op's 1 or 2, the other inputs then being folded in one after the other.
template <class D, class Op, int NIN, int LD, int ST>
__device__ __forceinline__ void chain_packs(const unsigned long long (&in)[kChainStreams], const unsigned long long (&out)[kChainStreams],
                                            int n_head, int n_out, unsigned int fed, size_t wg_off, unsigned int lane_off) {
  u32x4 v[NIN];
#pragma unroll
  for (int i = 0; i < NIN; ++i) v[i] = __builtin_amdgcn_raw_buffer_load_b128(whole_buffer((const char *)in[i] + wg_off), (int)lane_off, 0, LD);
  u32x4 cur;
  if (n_head == NIN) {
    cur = fold_pack<D, Op, NIN>(v);
  } else {
    cur = v[0];
    if constexpr (NIN >= 2) {
      if (n_head == 2) cur = fold_two<D, Op>(v[0], v[1]);
#pragma unroll
      for (int i = 1; i < NIN; ++i)
        if (i >= n_head) cur = ((fed >> i) & 1u) ? fold_two<D, Op>(v[i], cur) : fold_two<D, Op>(cur, v[i]);
    }
  }
#pragma unroll
  for (int j = 0; j < kChainStreams; ++j)
    if (j < n_out) __builtin_amdgcn_raw_buffer_store_b128(cur, whole_buffer((char *)out[j] + wg_off), (int)lane_off, 0, ST);
}

// ... and one of the few elements in front of the first and behind the last pack
template <class D, class Op, int NIN>
__device__ __forceinline__ void chain_elem(const unsigned long long (&in)[kChainStreams], const unsigned long long (&out)[kChainStreams],
                                           int n_head, int n_out, unsigned int fed, long long i) {
  typedef typename D::elem_t E;
  E x[NIN];
#pragma unroll
  for (int s = 0; s < NIN; ++s) x[s] = ((const E *)in[s])[i];
  E cur;
  if (n_head == NIN) {
    if constexpr (NIN == 1) cur = x[0];
    else cur = D::template elem<Op, NIN>(x);
  } else {
    cur = x[0];
    if constexpr (NIN >= 2) {
      if (n_head == 2) {
        const E two[2] = {x[0], x[1]};
        cur = D::template elem<Op, 2>(two);
      }
#pragma unroll
      for (int s = 1; s < NIN; ++s)
        if (s >= n_head) {
          const E two[2] = {((fed >> s) & 1u) ? x[s] : cur, ((fed >> s) & 1u) ? cur : x[s]};
          cur = D::template elem<Op, 2>(two);
        }
    }
  }
#pragma unroll
  for (int j = 0; j < kChainStreams; ++j)
    if (j < n_out) ((E *)out[j])[i] = cur;
}

// MEM (reduce_copy_kernel.h): kLaunchMemCached; kLaunchMemStreamWriteThrough (non-temporal loads, write-through
// stores); kLaunchMemStream for launches of fan-out copies (cached loads, non-temporal stores)
template <int DT, class Op, int MEM>
__global__ void __launch_bounds__(kBlock) graph_chains_kernel(const ChainsLaunch a) {
  typedef Dtype<DT> D;
  constexpr int kEpp = 16 / D::kElemBytes;
  D::wave_init();
  // (through the buffer instructions: the operands' addresses come out of memory, not out of the
  // kernel's pointer arguments, and a plain access through such an address would be a flat one; they
  // also take the operands that are only element-aligned)
  constexpr int kLdPolicy = MEM == pccl_dev::kLaunchMemStreamWriteThrough ? 2 : 0;  // nt
  constexpr int kStPolicy = MEM == pccl_dev::kLaunchMemCached ? 0 : MEM == pccl_dev::kLaunchMemStream ? 2 : kCachePolicySc1;
  const unsigned int b = blockIdx.x;
  int ci = 0;
#pragma unroll
  for (int k = 1; k < kLaunchChainGroups; ++k) ci += b >= a.first_wg[k] ? 1 : 0;  // (first_wg ascends)
  if (a.group > 1) {
    ci *= a.group;
    int more = 0;
#pragma unroll
    for (int k = 1; k < kLaunchChainsPerGroup; ++k)
      more += (k < a.group && ci + k < a.n_chains && b >= a.chains[ci + k].first_wg) ? 1 : 0;
    ci += more;
  }
  const LaunchChain *c = a.chains + ci;  // uniform: scalar loads
  const unsigned int k = b - c->first_wg;
  const unsigned int n_chunks = c->n_wg;
  const long long count = c->count;
  const int n_head = c->n_head, n_in = c->n_in, n_out = c->n_out;
  const unsigned int fed = c->fed;
  // (the whole row before anything is stored: the loads stay scalar)
  unsigned long long in[kChainStreams], out[kChainStreams];
#pragma unroll
  for (int i = 0; i < kChainStreams; ++i) {
    in[i] = c->in[i];
    out[i] = c->out[i];
  }
  const int uid = c->uid;
  const unsigned int chunk = a.rotate ? pccl_dev::rotated_chunk(k, n_chunks) : k;
  unsigned long long *trace = nullptr;
  if (a.trace && threadIdx.x == 0) {
    trace = a.trace + (size_t)b * kTraceWords;
    const unsigned long long now = wall_clock64();
    trace[kTraceWhat] = (unsigned long long)(unsigned int)uid | ((unsigned long long)chunk << 32) | ((unsigned long long)(b & 0xfffu) << 52);
    trace[kTraceClaimed] = now;
    trace[kTraceReady] = now;
  }
  // packs are cut so that output 0 is 16-byte aligned; the elements in front of the first pack and
  // behind the last one are left to the chain's last workgroup
  long long peel = (long long)((16 - (out[0] & 15)) & 15) / D::kElemBytes;
  if (peel > count) peel = count;
  const long long n_packs = (count - peel) / kEpp;
  // (read back into scalar registers: the compiler works this sum out on the vector unit, beside the lane's
  // pack number, and every operand's address would follow it there: a vector register pair per address that
  // each store then waits for the one before it to release)
  const size_t wg_off = (size_t)uniform64((unsigned long long)peel * D::kElemBytes + (unsigned long long)chunk * (kBlock * 16));
  const unsigned int lane_off = threadIdx.x * 16u;
  if ((long long)chunk * kBlock + threadIdx.x < n_packs) {
    switch (n_in) {
      case 1: chain_packs<D, Op, 1, kLdPolicy, kStPolicy>(in, out, n_head, n_out, fed, wg_off, lane_off); break;
      case 2: chain_packs<D, Op, 2, kLdPolicy, kStPolicy>(in, out, n_head, n_out, fed, wg_off, lane_off); break;
      case 3: chain_packs<D, Op, 3, kLdPolicy, kStPolicy>(in, out, n_head, n_out, fed, wg_off, lane_off); break;
      case 4: chain_packs<D, Op, 4, kLdPolicy, kStPolicy>(in, out, n_head, n_out, fed, wg_off, lane_off); break;
      case 5: chain_packs<D, Op, 5, kLdPolicy, kStPolicy>(in, out, n_head, n_out, fed, wg_off, lane_off); break;
      case 6: chain_packs<D, Op, 6, kLdPolicy, kStPolicy>(in, out, n_head, n_out, fed, wg_off, lane_off); break;
      case 7: chain_packs<D, Op, 7, kLdPolicy, kStPolicy>(in, out, n_head, n_out, fed, wg_off, lane_off); break;
      default: chain_packs<D, Op, 8, kLdPolicy, kStPolicy>(in, out, n_head, n_out, fed, wg_off, lane_off); break;
    }
  }
  if (k == n_chunks - 1 && threadIdx.x >= kBlock - kWave) {  // fewer than two packs' worth of elements: one per lane
    const long long tail_begin = peel + n_packs * kEpp, n_edge = peel + (count - tail_begin);
    const long long e = (long long)threadIdx.x - (kBlock - kWave);
    if (e < n_edge) {
      const long long i = e < peel ? e : tail_begin + (e - peel);
      switch (n_in) {
        case 1: chain_elem<D, Op, 1>(in, out, n_head, n_out, fed, i); break;
        case 2: chain_elem<D, Op, 2>(in, out, n_head, n_out, fed, i); break;
        case 3: chain_elem<D, Op, 3>(in, out, n_head, n_out, fed, i); break;
        case 4: chain_elem<D, Op, 4>(in, out, n_head, n_out, fed, i); break;
        case 5: chain_elem<D, Op, 5>(in, out, n_head, n_out, fed, i); break;
        case 6: chain_elem<D, Op, 6>(in, out, n_head, n_out, fed, i); break;
        case 7: chain_elem<D, Op, 7>(in, out, n_head, n_out, fed, i); break;
        default: chain_elem<D, Op, 8>(in, out, n_head, n_out, fed, i); break;
      }
    }
  }
  if (trace) {
    settle_stores();
    trace[kTraceDone] = wall_clock64();
  }
}

typedef void (*ChainsKernel)(const ChainsLaunch);
// The instances of one dtype; defined in graph_chains_inst_<dtype>.hip.  mem: a kLaunchMem* value.
template <int DT>
ChainsKernel chains_for_compute(int compute, int mem);

#define PCCL_CHAINS_KERNEL_OF(DT, OP)                                                             \
  (mem == pccl_dev::kLaunchMemStreamWriteThrough ? graph_chains_kernel<DT, OP, pccl_dev::kLaunchMemStreamWriteThrough> \
   : mem == pccl_dev::kLaunchMemStream           ? graph_chains_kernel<DT, OP, pccl_dev::kLaunchMemStream>             \
                                                 : graph_chains_kernel<DT, OP, pccl_dev::kLaunchMemCached>)

#define PCCL_DEFINE_CHAINS_FOR_COMPUTE(DT)                    \
  template <>                                                 \
  ChainsKernel chains_for_compute<DT>(int compute, int mem) { \
    switch (compute) {                                        \
      case PCCL_SUM: return PCCL_CHAINS_KERNEL_OF(DT, OpSum); \
      case PCCL_PROD: return PCCL_CHAINS_KERNEL_OF(DT, OpProd); \
      case PCCL_MIN: return PCCL_CHAINS_KERNEL_OF(DT, OpMin); \
      default: return PCCL_CHAINS_KERNEL_OF(DT, OpMax);       \
    }                                                         \
  }

}  // namespace pccl_queue
