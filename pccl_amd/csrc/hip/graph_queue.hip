// graph_queue.hip -- the op-batching path: a DAG of COPY / REDUCE ops lives on
// the device in the reference's GraphBufferLayout (include/base/operator.h:31-38)
// and ONE persistent kernel drains it; no launch per op.
//
// Protocol (the reference declares the structs, operator.h:7-38, but no code
// reads or writes them, so the protocol is defined here):
//   * an op is split into required_executors_ parts of about tile_bytes of
//     output; a ready-queue entry names (op_uid, part);
//   * workgroups claim entries by taking tickets from RingBuffer::head_; ticket
//     t waits until slot t has been published (RingBuffer::tail_ hands out slot
//     numbers to producers).  A slot is only ever published by a workgroup that
//     holds a smaller ticket, and tickets are only held by running workgroups,
//     so the drain cannot deadlock whatever the number of resident workgroups;
//   * the workgroup finishing the last part of an op decrements
//     pre_dependencies_ of each successor (32-bit atomic on the word at offset
//     12) and publishes the successors that reach zero;
//   * data moves between workgroups (possibly on different XCDs, whose L2s are not
//     coherent with each other) through device-coherent accesses: parts load and
//     store with sc1, wait for their stores, and only then touch the counters with
//     relaxed device-scope atomics.  An L2-wide write-back + invalidate per part
//     (what agent-scope release / acquire fences compile to) was measured to cost
//     about 100 us per part under load;
//   * per-op mutable state is restored by the op's last part and the run's
//     last workgroup rewinds the queue and re-publishes the initial entries,
//     so a finished graph is armed for its next run;
//   * every wait is bounded: when a wait exceeds spin_limit polls the kernel
//     raises the abort flag, all workgroups leave, and the host reports
//     PCCL_ERR_GRAPH instead of hanging.
#include <algorithm>
#include <cstring>
#include <mutex>
#include <vector>

#include "plugin_common.h"
#include "reduce_copy_device.h"

using namespace pccl_dev;
using pccl_host::fail;

namespace {

constexpr unsigned long long kEmptySlot = ~0ull;
constexpr long kDefaultTileBytes = 32 << 10;
constexpr unsigned int kDefaultSpinLimit = 1u << 21;  // a few seconds of polling

// Device-resident control block.  The reference's GraphBufferLayout is its
// first member, so the arena's base address is a GraphBufferLayout*.
struct GraphControl {
  pccl_graph_buffer_layout layout;
  pccl_operation_layout_header *headers;  // contiguous; layout.operators[i] == &headers[i]
  unsigned long long *slots;              // ready-queue storage, one pccl_queue_entry each
  const unsigned long long *initial;      // entries of the ops without dependencies
  unsigned int completed;                 // *layout.completed_operator
  unsigned int total;                     // *layout.total_operator
  unsigned int done_count;                // ops finished in the current run
  unsigned int exit_count;                // workgroups that have left the current run
  unsigned int abort;                     // set when a bounded wait gave up
  unsigned int spin_limit;
  int n_initial;
  int total_tiles;
};

__device__ __forceinline__ unsigned int *word12(pccl_operation_layout_header *h) {
  return (unsigned int *)((char *)h + 12);
}

// elements per part: the count split evenly, rounded up to 64 elements so that
// every part of an op keeps the alignment of the op's first element
__host__ __device__ inline long part_elems(long count, int parts) {
  long per = (count + parts - 1) / parts;
  return (per + 63) / 64 * 64;
}

template <class D, class Op, int NIN, bool ALIGNED>
__device__ __forceinline__ void run_part_body(const RcOperands &a, long head, long n_packs, long count) {
  constexpr int kEpp = 16 / D::kElemBytes;
  if (n_packs > 0) {
    RcOperands body;
    body.n_out = a.n_out;
#pragma unroll
    for (int k = 0; k < NIN; ++k) body.in[k] = a.in[k] + head * D::kElemBytes;
#pragma unroll
    for (int j = 0; j < PCCL_MAX_OUTPUTS; ++j)
      if (j < a.n_out) body.out[j] = a.out[j] + head * D::kElemBytes;
    // Every access of a part is device-coherent: its inputs may have been written
    // by a workgroup on another XCD moments ago, and its outputs may be read by one.
    constexpr int kUnroll = NIN >= 3 ? 1 : 2;
    body_packs<D, Op, NIN, kUnroll, ALIGNED, kMemCoherent, kMemCoherent>(body, n_packs, 0, 1);
  }
  if (threadIdx.x >= kBlock - kWave)
    edge_elems<D, Op, NIN, kMemCoherent>(a, head, head + n_packs * kEpp, count, (int)threadIdx.x - (kBlock - kWave));
  settle_stores();
}

template <class D, class Op, int NIN>
__device__ __forceinline__ void run_part_nin(const pccl_op_payload *pl, long lo, long count) {
  RcOperands a;
  a.n_out = pl->n_out_;
  a.out[0] = (char *)pl->chunks_[NIN].addr_ + lo * D::kElemBytes;
  // bits in which some stream's address differs from output 0's
  unsigned long long mis = 0;
#pragma unroll
  for (int k = 0; k < NIN; ++k) {
    a.in[k] = (const char *)pl->chunks_[k].addr_ + lo * D::kElemBytes;
    mis |= (unsigned long long)a.in[k] ^ (unsigned long long)a.out[0];
  }
#pragma unroll
  for (int j = 1; j < PCCL_MAX_OUTPUTS; ++j)
    if (j < a.n_out) {
      a.out[j] = (char *)pl->chunks_[NIN + j].addr_ + lo * D::kElemBytes;
      mis |= (unsigned long long)a.out[j] ^ (unsigned long long)a.out[0];
    }
  // same peel as the direct launch: make output 0 start on 16 bytes; the other
  // streams are 16-byte aligned after it exactly when they share its low bits
  long head = (long)((16 - ((unsigned long long)a.out[0] & 15)) & 15) / D::kElemBytes;
  if (head > count) head = count;
  const long n_packs = (count - head) / (16 / D::kElemBytes);
  const bool aligned = (mis & 15) == 0;
  if (aligned) run_part_body<D, Op, NIN, true>(a, head, n_packs, count);
  else run_part_body<D, Op, NIN, false>(a, head, n_packs, count);
}

template <int DT, class Op>
__device__ __forceinline__ void run_part(const pccl_op_payload *pl, long lo, long count) {
  typedef Dtype<DT> D;
  switch (pl->n_in_) {
    case 1: run_part_nin<D, Op, 1>(pl, lo, count); break;
    case 2: run_part_nin<D, Op, 2>(pl, lo, count); break;
    case 3: run_part_nin<D, Op, 3>(pl, lo, count); break;
    case 4: run_part_nin<D, Op, 4>(pl, lo, count); break;
    case 5: run_part_nin<D, Op, 5>(pl, lo, count); break;
    case 6: run_part_nin<D, Op, 6>(pl, lo, count); break;
    case 7: run_part_nin<D, Op, 7>(pl, lo, count); break;
    default: run_part_nin<D, Op, 8>(pl, lo, count); break;
  }
}

#define AGENT __HIP_MEMORY_SCOPE_AGENT

template <int DT, class Op>
__global__ void __launch_bounds__(kBlock) drain_graph_kernel(GraphControl *g) {
  __shared__ int s_ticket;
  __shared__ unsigned long long s_entry;
  __shared__ int s_last;
  pccl_ring_buffer *q = g->layout.ready_queues[0];
  unsigned long long *slots = g->slots;
  const int total_tiles = g->total_tiles;
  const unsigned int spin_limit = g->spin_limit;

  // Loop shape matters: thread 0's bookkeeping for the part just finished and its
  // claim of the next ticket sit in ONE conditional block per iteration, and the
  // loop exit is a scalar branch (readfirstlane).  With two thread-0 blocks (one
  // before the back edge, one after it) the compiler threads the jump between
  // them, the back edge becomes divergent, and the other lanes of thread 0's
  // wavefront run ahead into the next barrier while thread 0 is parked.
  pccl_operation_layout_header *h = nullptr;
  const pccl_op_payload *pl = nullptr;
  int parts = 0;
  for (;;) {
    if (threadIdx.x == 0) {
      if (h) {  // the part executed in the previous iteration is complete (barrier below):
        // every wavefront waited for its write-through stores before that barrier, so
        // the data is at the point of coherence and relaxed device-scope atomics are
        // enough to hand it over; no L2 write-back / invalidate is involved
        const int old = __hip_atomic_fetch_sub(&h->remaining_executors_, 1, __ATOMIC_RELAXED, AGENT);
        if (old == 1) {  // it was the op's last part
          __hip_atomic_store(&h->remaining_executors_, parts, __ATOMIC_RELAXED, AGENT);
          __hip_atomic_store(word12(h), pl->initial_word12_, __ATOMIC_RELAXED, AGENT);
          const int n_next = h->num_next_ops_;
          const int *next = h->next_op_uids_head_;
          for (int s = 0; s < n_next; ++s) {
            pccl_operation_layout_header *hs = &g->headers[next[s]];
            const unsigned int w = __hip_atomic_fetch_sub(word12(hs), 1u, __ATOMIC_RELAXED, AGENT);
            if ((w & 0xffu) == 1u) {  // last dependency gone: publish all its parts
              const int r = hs->required_executors_;
              const int pos = __hip_atomic_fetch_add(&q->tail_, r, __ATOMIC_RELAXED, AGENT);
              for (int p = 0; p < r; ++p) {
                const unsigned long long e = (unsigned long long)(unsigned int)next[s] | ((unsigned long long)p << 32);
                __hip_atomic_store(&slots[pos + p], e, __ATOMIC_RELAXED, AGENT);
              }
            }
          }
          __hip_atomic_fetch_add(&g->done_count, 1u, __ATOMIC_RELAXED, AGENT);
        }
      }
      int t = total_tiles;  // "leave"
      if (__hip_atomic_load(&g->abort, __ATOMIC_RELAXED, AGENT) == 0)
        t = __hip_atomic_fetch_add(&q->head_, 1, __ATOMIC_RELAXED, AGENT);
      if (t < total_tiles) {
        if (t == 0) __hip_atomic_store(&g->completed, 0u, __ATOMIC_RELAXED, AGENT);
        unsigned long long e;
        unsigned int spins = 0;
        for (;;) {
          e = __hip_atomic_load(&slots[t], __ATOMIC_RELAXED, AGENT);
          if (e != kEmptySlot) break;
          __builtin_amdgcn_s_sleep(2);
          if ((++spins & 63u) == 0 &&
              (spins >= spin_limit || __hip_atomic_load(&g->abort, __ATOMIC_RELAXED, AGENT) != 0)) {
            __hip_atomic_store(&g->abort, 1u, __ATOMIC_RELAXED, AGENT);
            t = total_tiles;
            break;
          }
        }
        if (t < total_tiles) {
          __hip_atomic_store(&slots[t], kEmptySlot, __ATOMIC_RELAXED, AGENT);  // slot ready for the next run
          s_entry = e;
        }
      }
      s_ticket = t;
    }
    __syncthreads();
    if (__builtin_amdgcn_readfirstlane(s_ticket) >= total_tiles) break;
    const int uid = __builtin_amdgcn_readfirstlane((int)(s_entry & 0xffffffffu));
    const int part = __builtin_amdgcn_readfirstlane((int)(s_entry >> 32));
    h = &g->headers[uid];
    pl = (const pccl_op_payload *)h->op_buffer_;
    parts = h->required_executors_;
    const long count = pl->chunks_[0].num_elems_;
    const long per = part_elems(count, parts);
    const long lo = (long)part * per;
    long n = count - lo;
    if (n > per) n = per;
    if (n > 0) run_part<DT, Op>(pl, lo, n);
    // every store of this part is issued and complete at workgroup scope before
    // thread 0 releases it at the top of the next iteration; also keeps s_entry /
    // s_ticket from being rewritten while other wavefronts still read them
    __syncthreads();
  }

  // leave: the last workgroup out re-arms the graph for the next run
  if (threadIdx.x == 0) {
    settle_stores();  // this workgroup's counter updates land before it counts as gone
    const unsigned int e = __hip_atomic_fetch_add(&g->exit_count, 1u, __ATOMIC_RELAXED, AGENT);
    s_last = (e == gridDim.x - 1);
  }
  __syncthreads();
  if (!__builtin_amdgcn_readfirstlane(s_last)) return;
  if (__hip_atomic_load(&g->abort, __ATOMIC_RELAXED, AGENT) != 0) {
    if (threadIdx.x == 0) {
      __hip_atomic_store(&g->completed, __hip_atomic_load(&g->done_count, __ATOMIC_RELAXED, AGENT),
                         __ATOMIC_RELAXED, AGENT);
      __hip_atomic_store(&g->exit_count, 0u, __ATOMIC_RELAXED, AGENT);
    }
    return;  // state is inconsistent; the host re-uploads it before the next run
  }
  const int n_initial = g->n_initial;
  for (int i = threadIdx.x; i < n_initial; i += kBlock)
    __hip_atomic_store(&slots[i], g->initial[i], __ATOMIC_RELAXED, AGENT);
  if (threadIdx.x == 0) {
    __hip_atomic_store(&g->completed, __hip_atomic_load(&g->done_count, __ATOMIC_RELAXED, AGENT),
                       __ATOMIC_RELAXED, AGENT);
    __hip_atomic_store(&g->done_count, 0u, __ATOMIC_RELAXED, AGENT);
    __hip_atomic_store(&g->exit_count, 0u, __ATOMIC_RELAXED, AGENT);
    __hip_atomic_store(&q->head_, 0, __ATOMIC_RELAXED, AGENT);
    __hip_atomic_store(&q->tail_, n_initial, __ATOMIC_RELAXED, AGENT);
  }
}

typedef void (*DrainKernel)(GraphControl *);

template <int DT>
DrainKernel drain_for_compute(int compute) {
  switch (compute) {
    case PCCL_SUM: return drain_graph_kernel<DT, OpSum>;
    case PCCL_PROD: return drain_graph_kernel<DT, OpProd>;
    case PCCL_MIN: return drain_graph_kernel<DT, OpMin>;
    default: return drain_graph_kernel<DT, OpMax>;
  }
}

DrainKernel drain_for(int dtype, int compute) {
  switch (dtype) {
    case PCCL_F32: return drain_for_compute<PCCL_F32>(compute);
    case PCCL_I32: return drain_for_compute<PCCL_I32>(compute);
    case PCCL_BF16: return drain_for_compute<PCCL_BF16>(compute);
    default: return drain_for_compute<PCCL_F16>(compute);
  }
}

// ---- host side ----------------------------------------------------------------

struct Graph {
  char *dev = nullptr;          // device arena; starts with GraphControl
  std::vector<char> image;      // pristine host copy of the arena
  size_t payload_off = 0;       // arena offset of the payload array
  int n_ops = 0;
  int total_tiles = 0;
  int n_wg = 0;
  int device = 0;
  DrainKernel kernel = nullptr;
  std::mutex mu;
};

constexpr size_t kPayloadStride = 256;  // sizeof(pccl_op_payload) == 248, padded

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

int elem_bytes(int dtype) { return (dtype == PCCL_F32 || dtype == PCCL_I32) ? 4 : 2; }

}  // namespace

extern "C" {

int pccl_hip_graph_create(const pccl_op_desc *ops, int n_ops, long tile_bytes, void **graph) {
  pccl_host::clear_error();
  if (!graph) return fail(PCCL_ERR_INVALID_ARG, "graph_create: graph is null");
  *graph = nullptr;
  if (n_ops < 0 || (n_ops > 0 && !ops)) return fail(PCCL_ERR_INVALID_ARG, "graph_create: bad op array");
  if (tile_bytes < 0) return fail(PCCL_ERR_INVALID_ARG, "graph_create: tile_bytes %ld < 0", tile_bytes);
  if (tile_bytes == 0) tile_bytes = kDefaultTileBytes;
  tile_bytes = std::max<long>(tile_bytes, 1024);

  // ---- validate; one (dtype, compute) pair for all REDUCE ops --------------
  int g_dtype = -1, g_compute = -1;
  std::vector<int> n_succ(n_ops, 0), n_pred(n_ops, 0), parts(n_ops, 1);
  size_t n_edges = 0;
  long long tiles = 0;
  for (int i = 0; i < n_ops; ++i) {
    const pccl_op_desc &o = ops[i];
    if (o.op_uid != i) return fail(PCCL_ERR_GRAPH, "op %d: op_uid %d is not its index (uids are dense from 0)", i, o.op_uid);
    if (o.primitive != PCCL_COPY && o.primitive != PCCL_REDUCE)
      return fail(PCCL_ERR_UNSUPPORTED, "op %d: primitive %d is not COPY or REDUCE", i, o.primitive);
    if (o.dtype > PCCL_F16) return fail(PCCL_ERR_UNSUPPORTED, "op %d: unknown dtype code %d", i, o.dtype);
    if (o.compute > PCCL_MAX) return fail(PCCL_ERR_UNSUPPORTED, "op %d: unknown compute code %d", i, o.compute);
    if (o.n_in < 1 || o.n_in > PCCL_MAX_INPUTS || o.n_out < 1 || o.n_out > PCCL_MAX_OUTPUTS ||
        o.n_in + o.n_out > PCCL_MAX_OP_CHUNKS)
      return fail(PCCL_ERR_INVALID_ARG, "op %d: n_in %d / n_out %d (each 1..8, at most 10 operands in all)", i, o.n_in, o.n_out);
    if (o.primitive == PCCL_COPY && o.n_in != 1)
      return fail(PCCL_ERR_INVALID_ARG, "op %d: COPY takes exactly one input", i);
    if (o.count < 0) return fail(PCCL_ERR_INVALID_ARG, "op %d: count %ld < 0", i, o.count);
    const int es = elem_bytes(o.dtype);
    for (int k = 0; k < o.n_in; ++k) {
      if (!o.ins[k] && o.count) return fail(PCCL_ERR_INVALID_ARG, "op %d: input %d is null", i, k);
      if ((uintptr_t)o.ins[k] % es) return fail(PCCL_ERR_MISALIGNED, "op %d: input %d not %d-byte aligned", i, k, es);
    }
    for (int k = 0; k < o.n_out; ++k) {
      if (!o.outs[k] && o.count) return fail(PCCL_ERR_INVALID_ARG, "op %d: output %d is null", i, k);
      if ((uintptr_t)o.outs[k] % es) return fail(PCCL_ERR_MISALIGNED, "op %d: output %d not %d-byte aligned", i, k, es);
    }
    if (o.n_in > 1) {
      if (g_dtype < 0) { g_dtype = o.dtype; g_compute = o.compute; }
      else if (g_dtype != o.dtype || g_compute != o.compute)
        return fail(PCCL_ERR_UNSUPPORTED, "op %d: a graph holds REDUCE ops of one (dtype, compute) pair only", i);
    }
    if (o.n_deps < 0 || (o.n_deps > 0 && !o.deps)) return fail(PCCL_ERR_GRAPH, "op %d: bad dependency list", i);
    if (o.n_deps > 255) return fail(PCCL_ERR_GRAPH, "op %d: %d dependencies exceed pre_dependencies_ (unsigned char)", i, o.n_deps);
    for (int d = 0; d < o.n_deps; ++d) {
      const int u = o.deps[d];
      if (u < 0 || u >= n_ops || u == i) return fail(PCCL_ERR_GRAPH, "op %d: dependency %d is not another op", i, u);
      ++n_succ[u];
    }
    n_pred[i] = o.n_deps;
    n_edges += (size_t)o.n_deps;
    const long bytes = o.count * es;
    long p = (bytes + tile_bytes - 1) / tile_bytes;
    parts[i] = (int)std::max<long>(1, std::min<long>(p, 1 << 20));
    tiles += parts[i];
  }
  for (int i = 0; i < n_ops; ++i)
    if (n_succ[i] > 255) return fail(PCCL_ERR_GRAPH, "op %d: %d successors exceed num_next_ops_ (unsigned char)", i, n_succ[i]);
  if (tiles > (1ll << 30)) return fail(PCCL_ERR_GRAPH, "graph needs %lld queue entries", tiles);
  // copy-only graphs: element size of the ops decides nothing but alignment assumptions
  if (g_dtype < 0) { g_dtype = PCCL_BF16; g_compute = PCCL_SUM; }

  // ---- acyclicity (Kahn) -----------------------------------------------------
  std::vector<int> succ_start(n_ops + 1, 0);
  for (int i = 0; i < n_ops; ++i) succ_start[i + 1] = succ_start[i] + n_succ[i];
  std::vector<int> succ(n_edges ? n_edges : 1), fill(n_ops, 0);
  for (int i = 0; i < n_ops; ++i)
    for (int d = 0; d < ops[i].n_deps; ++d) {
      const int u = ops[i].deps[d];
      succ[succ_start[u] + fill[u]++] = i;
    }
  {
    std::vector<int> indeg(n_pred), stack;
    for (int i = 0; i < n_ops; ++i) if (!indeg[i]) stack.push_back(i);
    int seen = 0;
    while (!stack.empty()) {
      const int u = stack.back();
      stack.pop_back();
      ++seen;
      for (int e = succ_start[u]; e < succ_start[u + 1]; ++e)
        if (--indeg[succ[e]] == 0) stack.push_back(succ[e]);
    }
    if (seen != n_ops) return fail(PCCL_ERR_GRAPH, "dependency graph has a cycle (%d of %d ops reachable)", seen, n_ops);
  }

  // ---- arena layout ----------------------------------------------------------
  size_t off = align_up(sizeof(GraphControl), 256);
  const size_t off_opptr = off;   off = align_up(off + sizeof(void *) * (size_t)std::max(n_ops, 1), 256);
  const size_t off_hdr = off;     off = align_up(off + sizeof(pccl_operation_layout_header) * (size_t)std::max(n_ops, 1), 256);
  const size_t off_payload = off; off = align_up(off + kPayloadStride * (size_t)std::max(n_ops, 1), 256);
  const size_t off_succ = off;    off = align_up(off + sizeof(int) * std::max<size_t>(n_edges, 1), 256);
  const size_t off_ring = off;    off = align_up(off + sizeof(pccl_ring_buffer), 256);
  const size_t off_qptr = off;    off = align_up(off + sizeof(void *), 256);
  const size_t off_slots = off;   off = align_up(off + 8 * (size_t)std::max<long long>(tiles, 1), 256);
  const size_t off_init = off;    off = align_up(off + 8 * (size_t)std::max<long long>(tiles, 1), 256);
  const size_t arena_bytes = off;

  Graph *G = new Graph();
  G->n_ops = n_ops;
  G->total_tiles = (int)tiles;
  G->payload_off = off_payload;
  G->kernel = drain_for(g_dtype, g_compute);
  if (hipGetDevice(&G->device) != hipSuccess) { delete G; return fail(PCCL_ERR_NO_DEVICE, "no current device"); }
  hipError_t e = hipMalloc((void **)&G->dev, arena_bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    delete G;
    return fail(PCCL_ERR_NOMEM, "hipMalloc(%zu) for the op graph: %s", arena_bytes, hipGetErrorString(e));
  }
  G->image.assign(arena_bytes, 0);
  char *img = G->image.data();
  char *dev = G->dev;

  GraphControl *C = (GraphControl *)img;
  C->layout.completed_operator = (unsigned int *)(dev + offsetof(GraphControl, completed));
  C->layout.total_operator = (unsigned int *)(dev + offsetof(GraphControl, total));
  C->layout.operators = (pccl_operation_layout_header **)(dev + off_opptr);
  C->layout.num_operators = (unsigned int)n_ops;
  C->layout.ready_queues = (pccl_ring_buffer **)(dev + off_qptr);
  C->layout.num_queues = 1;
  C->headers = (pccl_operation_layout_header *)(dev + off_hdr);
  C->slots = (unsigned long long *)(dev + off_slots);
  C->initial = (const unsigned long long *)(dev + off_init);
  C->completed = 0;
  C->total = (unsigned int)n_ops;
  C->spin_limit = kDefaultSpinLimit;
  C->total_tiles = (int)tiles;

  *(pccl_ring_buffer **)(img + off_qptr) = (pccl_ring_buffer *)(dev + off_ring);
  pccl_ring_buffer *R = (pccl_ring_buffer *)(img + off_ring);
  R->producer_ = 0;  // executor ids are the host layer's; one executor produces and consumes
  R->consumer_ = 0;
  R->elem_size_ = (int)sizeof(pccl_queue_entry);
  R->max_num_elems_ = (int)std::max<long long>(tiles, 1);
  R->max_flush_time_ = 0;  // producer and consumer share one address space: nothing to flush
  R->producer_buffer_ = dev + off_slots;
  R->consumer_buffer_ = dev + off_slots;

  unsigned long long *slots = (unsigned long long *)(img + off_slots);
  unsigned long long *initial = (unsigned long long *)(img + off_init);
  for (long long t = 0; t < std::max<long long>(tiles, 1); ++t) slots[t] = kEmptySlot;
  int n_initial = 0;

  for (int i = 0; i < n_ops; ++i) {
    const pccl_op_desc &o = ops[i];
    ((pccl_operation_layout_header **)(img + off_opptr))[i] =
        (pccl_operation_layout_header *)(dev + off_hdr) + i;
    pccl_operation_layout_header *h = (pccl_operation_layout_header *)(img + off_hdr) + i;
    h->op_uid_ = i;
    h->required_executors_ = parts[i];
    h->remaining_executors_ = parts[i];
    h->pre_dependencies_ = (unsigned char)n_pred[i];
    h->executor_type_ = 0;
    h->op_size_ = (unsigned char)(8 + sizeof(pccl_chunk_meta) * (size_t)(o.n_in + o.n_out));
    h->num_next_ops_ = (unsigned char)n_succ[i];
    h->op_buffer_ = dev + off_payload + kPayloadStride * (size_t)i;
    h->next_op_uids_head_ = (int *)(dev + off_succ) + succ_start[i];
    pccl_op_payload *pl = (pccl_op_payload *)(img + off_payload + kPayloadStride * (size_t)i);
    pl->primitive_ = o.primitive;
    pl->compute_ = o.compute;
    pl->n_in_ = o.n_in;
    pl->n_out_ = o.n_out;
    memcpy(&pl->initial_word12_, (char *)h + 12, 4);
    for (int k = 0; k < o.n_in; ++k) pl->chunks_[k] = pccl_chunk_meta{o.dtype, (void *)o.ins[k], o.count};
    for (int k = 0; k < o.n_out; ++k) pl->chunks_[o.n_in + k] = pccl_chunk_meta{o.dtype, o.outs[k], o.count};
    if (n_pred[i] == 0)
      for (int p = 0; p < parts[i]; ++p)
        initial[n_initial++] = (unsigned long long)(unsigned int)i | ((unsigned long long)p << 32);
  }
  if (n_edges) memcpy(img + off_succ, succ.data(), sizeof(int) * n_edges);
  for (int t = 0; t < n_initial; ++t) slots[t] = initial[t];
  R->head_ = 0;
  R->tail_ = n_initial;
  C->n_initial = n_initial;

  // launch width: enough workgroups to fill the chip, never more than entries
  int occ = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void *)G->kernel, kBlock, 0) != hipSuccess || occ < 1) {
    (void)hipGetLastError();
    occ = 4;
  }
  occ = std::min(occ, 8);
  const long long cap = (long long)pccl_host::compute_units() * occ;
  G->n_wg = (int)std::max<long long>(1, std::min<long long>(tiles, cap));

  e = hipMemcpy(dev, img, arena_bytes, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(dev);
    delete G;
    return fail(PCCL_ERR_HIP, "uploading the op graph: %s", hipGetErrorString(e));
  }
  *graph = G;
  return PCCL_OK;
}

int pccl_hip_graph_run(void *graph, void *stream) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_run: graph is null");
  if (G->total_tiles == 0) return PCCL_OK;
  hipLaunchKernelGGL(G->kernel, dim3((unsigned)G->n_wg), dim3(kBlock), 0, (hipStream_t)stream, (GraphControl *)G->dev);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(PCCL_ERR_HIP, "graph_run launch failed: %s", hipGetErrorString(e));
  return PCCL_OK;
}

int pccl_hip_graph_status(void *graph, void *stream, unsigned int *completed, unsigned int *total) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_status: graph is null");
  PCCL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
  GraphControl c;
  PCCL_HIP_CHECK(hipMemcpy(&c, G->dev, sizeof(c), hipMemcpyDeviceToHost));
  if (completed) *completed = c.completed;
  if (total) *total = c.total;
  if (c.abort) {
    // put the pristine state back so that the graph can be used again
    std::lock_guard<std::mutex> lock(G->mu);
    PCCL_HIP_CHECK(hipMemcpy(G->dev, G->image.data(), G->image.size(), hipMemcpyHostToDevice));
    return fail(PCCL_ERR_GRAPH, "drain gave up: a queue slot was not published within the spin limit "
                                "(%u of %u ops had completed); graph state was reset", c.completed, c.total);
  }
  return PCCL_OK;
}

int pccl_hip_graph_rebind(void *graph, const void *old_base, const void *new_base, long nbytes, void *stream) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_rebind: graph is null");
  if (nbytes < 0) return fail(PCCL_ERR_INVALID_ARG, "graph_rebind: nbytes %ld < 0", nbytes);
  if (((uintptr_t)old_base ^ (uintptr_t)new_base) & 3)
    return fail(PCCL_ERR_MISALIGNED, "graph_rebind: bases differ in their low address bits");
  if (G->n_ops == 0 || nbytes == 0 || old_base == new_base) return PCCL_OK;
  std::lock_guard<std::mutex> lock(G->mu);
  const uintptr_t lo = (uintptr_t)old_base, hi = lo + (uintptr_t)nbytes;
  char *payloads = G->image.data() + G->payload_off;
  for (int i = 0; i < G->n_ops; ++i) {
    pccl_op_payload *pl = (pccl_op_payload *)(payloads + kPayloadStride * (size_t)i);
    const int nc = pl->n_in_ + pl->n_out_;
    for (int k = 0; k < nc; ++k) {
      const uintptr_t a = (uintptr_t)pl->chunks_[k].addr_;
      if (a >= lo && a < hi) pl->chunks_[k].addr_ = (void *)((uintptr_t)new_base + (a - lo));
    }
  }
  // ordered after earlier runs on `stream`; the source is pageable host memory,
  // so the call returns once the bytes are staged
  PCCL_HIP_CHECK(hipMemcpyAsync(G->dev + G->payload_off, payloads, kPayloadStride * (size_t)G->n_ops,
                                hipMemcpyHostToDevice, (hipStream_t)stream));
  return PCCL_OK;
}

int pccl_hip_graph_info(void *graph, void **device_layout, int *n_tiles, int *n_workgroups) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_info: graph is null");
  if (device_layout) *device_layout = G->dev;
  if (n_tiles) *n_tiles = G->total_tiles;
  if (n_workgroups) *n_workgroups = G->n_wg;
  return PCCL_OK;
}

int pccl_hip_graph_set_spin_limit(void *graph, unsigned int polls) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_set_spin_limit: graph is null");
  if (polls < 64) polls = 64;
  std::lock_guard<std::mutex> lock(G->mu);
  ((GraphControl *)G->image.data())->spin_limit = polls;
  PCCL_HIP_CHECK(hipMemcpy(G->dev + offsetof(GraphControl, spin_limit), &polls, sizeof(polls), hipMemcpyHostToDevice));
  return PCCL_OK;
}

int pccl_hip_graph_destroy(void *graph) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return PCCL_OK;
  hipError_t e = hipFree(G->dev);
  delete G;
  if (e != hipSuccess) return fail(PCCL_ERR_HIP, "hipFree of the op graph: %s", hipGetErrorString(e));
  return PCCL_OK;
}

}  // extern "C"
